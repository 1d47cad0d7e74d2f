"""GPU parity: router softmax/top-k and expert alignment vs the CPU oracle (C ABI path)."""
import numpy as np
import pytest
import torch

from oracle import moe_gating as og
from test_oracle_gating import check_align_invariants

pytestmark = pytest.mark.gpu


def _topk(logits_cpu, k, dev, renorm=True):
    from dlcompiler_amd.kernels.moe_gating import moe_topk_softmax

    w, ids = moe_topk_softmax(logits_cpu.to(dev), k, renormalize=renorm)
    assert w.dtype == torch.float32 and ids.dtype == torch.int32
    return w.cpu(), ids.cpu()


@pytest.mark.parametrize("T,E,k", [(16384, 64, 6), (128, 4, 2), (4096, 64, 8), (1, 64, 6),
                                   (77, 8, 2), (333, 60, 6), (100, 128, 8), (50, 160, 6),
                                   (19, 256, 16), (5, 3, 3)])
@pytest.mark.parametrize("renorm", [True, False])
def test_topk_softmax_parity(dev, T, E, k, renorm):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn((T, E), generator=g)
    w, ids = _topk(logits, k, dev, renorm)
    rw, rids = og.topk_softmax(logits, k, renormalize=renorm)
    assert torch.equal(ids, rids)                               # bit-exact indices
    torch.testing.assert_close(w, rw, rtol=1e-6, atol=0)        # north-star: 1e-6 relative


# the reference's fused gate kernel in its own output form (topk_gating_fwd_part1.py:63-81):
# full softmax gates [S, E] and one-hot masks [k, S, E] int64
@pytest.mark.parametrize("S,E,k,dtype", [(16384, 64, 6, torch.float32), (4096, 64, 8, torch.float32),
                                         (333, 60, 6, torch.float32), (50, 160, 6, torch.float32),
                                         (19, 256, 16, torch.float32), (5, 3, 3, torch.float32),
                                         (777, 64, 2, torch.float16)])
def test_topk_gating_part1_outputs(dev, S, E, k, dtype):
    from dlcompiler_amd.kernels.moe_gating import moe_topk_softmax
    from dlcompiler_amd.kernels.topk_gating_fwd_part1 import call

    g = torch.Generator().manual_seed(S + E)
    logits = torch.randn((S, E), generator=g).to(dtype)
    gates, masks = call(logits.to(dev), k)
    assert gates.shape == (S, E) and gates.dtype == dtype
    assert masks.shape == (k, S, E) and masks.dtype == torch.int64
    rg, rm = og.topk_gating_part1(logits, k)
    tol = dict(rtol=2e-6, atol=0) if dtype == torch.float32 else dict(rtol=2e-3, atol=1e-7)
    torch.testing.assert_close(gates.cpu(), rg, **tol)
    # the selection is unique where the top-(k+1) gate values of the oracle are distinct (it
    # selects on rounded probabilities, the kernel on the logits)
    top = torch.topk(rg.float(), min(k + 1, E), dim=-1).values
    unique = (top[:, :-1] != top[:, 1:]).all(-1)
    assert unique.float().mean() > 0.95
    m = masks.cpu()
    assert torch.equal(m[:, unique], rm[:, unique])
    assert (m.sum(-1) == 1).all() and (m.sum(0) <= 1).all()
    # the index form and the one-hot form come from one kernel and say the same
    w, ids = moe_topk_softmax(logits.to(dev), k, renormalize=False)
    assert torch.equal(m.argmax(-1).t().to(torch.int32), ids.cpu())
    assert torch.equal(torch.gather(gates.float().cpu(), 1, ids.cpu().long()),
                       w.cpu()) or dtype != torch.float32


def test_topk_ties_resolve_to_lowest_index(dev):
    logits = torch.zeros((40, 64))
    logits[1, 10:20] = 2.0
    logits[2] = torch.arange(64).float().flip(0)
    logits[3, ::2] = 1.0
    logits[4, 5] = -0.0
    g = torch.Generator().manual_seed(9)
    logits[8:] = torch.randint(-2, 3, (32, 64), generator=g).float()   # many ties
    w, ids = _topk(logits, 6, dev)
    rw, rids = og.topk_softmax(logits, 6)
    assert ids[0].tolist() == [0, 1, 2, 3, 4, 5]
    assert ids[1].tolist() == [10, 11, 12, 13, 14, 15]
    assert ids[3].tolist() == [0, 2, 4, 6, 8, 10]
    assert ids[4].tolist() == [0, 1, 2, 3, 4, 5]
    assert torch.equal(ids, rids)
    torch.testing.assert_close(w, rw, rtol=1e-6, atol=0)


def test_topk_strided_and_extreme_logits(dev):
    from dlcompiler_amd.kernels.moe_gating import moe_topk_softmax

    g = torch.Generator().manual_seed(4)
    wide = torch.randn((64, 200), generator=g) * 30.0           # exp would overflow unshifted
    view = wide[:, 3:67]
    w, ids = moe_topk_softmax(wide.to(dev)[:, 3:67], 6)
    rw, rids = og.topk_softmax(view.contiguous(), 6)
    assert torch.equal(ids.cpu(), rids)
    torch.testing.assert_close(w.cpu(), rw, rtol=1e-6, atol=1e-30)


def _align(ids_cpu, block, E, dev):
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size

    out = moe_align_block_size(ids_cpu.to(dev), block, E, return_counts=True)
    return [t.cpu() for t in out]


@pytest.mark.parametrize("T,k,E,block", [(16384, 6, 64, 64), (4096, 6, 64, 64), (128, 2, 4, 16),
                                         (1, 6, 64, 64), (7, 3, 5, 1), (1000, 8, 256, 128),
                                         (3000, 4, 60, 32), (2048, 1, 2, 64), (513, 2, 160, 8),
                                         (140000, 4, 32, 64)])  # > 256 chunks: separate scan kernel
def test_align_bit_exact(dev, T, k, E, block):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn((T, E), generator=g)
    _, ids = og.topk_softmax(logits, k)
    s, e, tot, cnt = _align(ids, block, E, dev)
    rs, re_, rtot, rcnt = og.align_block_size(ids, block, E)
    assert torch.equal(cnt, rcnt) and torch.equal(tot, rtot)
    assert torch.equal(e, re_)
    assert torch.equal(s, rs)
    check_align_invariants(ids.flatten().numpy(), block, E, s, e, tot.item(), cnt)
    # reference view of the same data: exp_start/exp_end (fused_moe.py:271-275)
    start, end = og.start_end(ids, E)
    assert torch.equal(end - start, cnt.long())


def test_align_empty_skewed_and_dropped(dev):
    s, e, tot, cnt = _align(torch.zeros((0, 6), dtype=torch.int32), 64, 64, dev)
    assert tot.item() == 0 and cnt.sum() == 0 and (s == 0).all() and (e == -1).all()
    # every slot on one expert; and a list with ids owned by another shard
    for ids in [torch.full((5000, 2), 3, dtype=torch.int32),
                torch.tensor([[0, 70], [-1, 1], [1, 64], [63, 0]], dtype=torch.int32)]:
        out = _align(ids, 64, 64, dev)
        ref = og.align_block_size(ids, 64, 64)
        for a, b in zip(out, ref):
            assert torch.equal(a, b)


def test_align_is_deterministic(dev):
    g = torch.Generator().manual_seed(11)
    ids = torch.randint(0, 64, (16384, 6), generator=g, dtype=torch.int32)
    first = _align(ids, 64, 64, dev)
    for _ in range(3):
        again = _align(ids, 64, 64, dev)
        assert all(torch.equal(a, b) for a, b in zip(first, again))


def test_end_to_end_config2(dev):
    # benchmark configuration 2: logits fp32 [16384, 64] ~ N(0,1) seed 1, k = 6, block 64
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size, moe_topk_softmax

    g = torch.Generator().manual_seed(1)
    logits = torch.randn((16384, 64), generator=g)
    w, ids = moe_topk_softmax(logits.to(dev), 6)
    s, e, tot = moe_align_block_size(ids, 64, 64)
    rw, rids = og.topk_softmax(logits, 6)
    rs, re_, rtot, _ = og.align_block_size(rids, 64, 64)
    assert torch.equal(ids.cpu(), rids) and torch.equal(s.cpu(), rs)
    assert torch.equal(e.cpu(), re_) and tot.item() == rtot.item()
    torch.testing.assert_close(w.cpu(), rw, rtol=1e-6, atol=0)
    np.testing.assert_allclose(w.cpu().sum(-1).numpy(), 1.0, atol=3e-7)


@pytest.mark.parametrize("T,E,k,block", [(16384, 64, 6, 64), (1, 64, 6, 64), (127, 8, 2, 16),
                                         (128, 60, 6, 64), (129, 64, 8, 128), (333, 160, 6, 32),
                                         (5000, 256, 16, 64), (32768, 16, 4, 64), (0, 64, 6, 64),
                                         (63, 64, 6, 64), (65, 64, 6, 64), (16385, 64, 6, 64),  # 64- / 128-token chunks
                                         (40000, 64, 6, 64)])   # the last one: the two-call path
@pytest.mark.parametrize("renorm", [True, False])
def test_fused_router_and_alignment_equals_the_two_calls(dev, T, E, k, block, renorm):
    from dlcompiler_amd.kernels.moe_gating import (moe_align_block_size, moe_topk_softmax,
                                                   moe_topk_softmax_align)

    g = torch.Generator().manual_seed(T + E)
    logits = torch.randn((T, E), generator=g).to(dev)
    if T > 3:
        logits[2] = 0.0                                       # a row of ties
    w, ids, sorted_ids, expert_ids, npad = moe_topk_softmax_align(logits, k, block, renormalize=renorm)
    rw, rids = moe_topk_softmax(logits, k, renormalize=renorm)
    rs, re_, rn = moe_align_block_size(rids, block, E)
    assert w.dtype == torch.float32 and ids.dtype == torch.int32 and w.shape == (T, k)
    assert torch.equal(ids, rids) and torch.equal(w, rw)
    assert torch.equal(npad, rn) and torch.equal(sorted_ids, rs) and torch.equal(expert_ids, re_)
    if T > 0:   # and against the oracle, not only against the other native path
        ow, oids = og.topk_softmax(logits.cpu(), k, renormalize=renorm)
        assert torch.equal(ids.cpu(), oids)
        os_, oe, otot, _ = og.align_block_size(oids, block, E)
        assert torch.equal(sorted_ids.cpu(), os_) and torch.equal(expert_ids.cpu(), oe)
        assert int(npad.item()) == int(otot.item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k", [(1000, 64, 6), (333, 128, 8), (77, 256, 4), (50, 60, 3), (40, 100, 2)])
def test_sixteen_bit_logits_are_read_as_they_are(dev, dtype, T, E, k):
    """bf16 / fp16 router logits go to the kernels unconverted (the reference's gate kernel takes
    them too, topk_gating_fwd_part1.py:44-46): same results, bit for bit, as the fp32 copy."""
    from dlcompiler_amd.kernels.moe_gating import moe_topk_softmax, moe_topk_softmax_align

    g = torch.Generator().manual_seed(T + E)
    wide = torch.randn((T, E + 8), generator=g).to(dtype).to(dev)
    for logits in (wide[:, :E].contiguous(), wide[:, :E]):       # vector rows, and a strided view
        ref = moe_topk_softmax(logits.float(), k, True, return_probs=True)
        got = moe_topk_softmax(logits, k, True, return_probs=True)
        for a, b in zip(ref, got):
            assert torch.equal(a, b)
        ref = moe_topk_softmax_align(logits.float(), k, 64, return_counts=True)
        got = moe_topk_softmax_align(logits, k, 64, return_counts=True)
        for a, b in zip(ref, got):
            assert torch.equal(a, b)
    # and against the oracle on the same 16-bit values
    rw, rids = og.topk_softmax(wide[:, :E].cpu(), k)
    w, ids = moe_topk_softmax(wide[:, :E], k)
    assert torch.equal(ids.cpu(), rids)
    torch.testing.assert_close(w.cpu(), rw, rtol=1e-6, atol=0)


@pytest.mark.parametrize("T,E,k,block", [(4096, 64, 6, 128), (300, 8, 2, 16), (1, 4, 1, 64)])
def test_int64_routing_ids_are_read_as_they_are(dev, T, E, k, block):
    """torch.topk hands over int64 ids and the reference's fused_moe takes them
    (fused_moe.py:296-320): the alignment reads either width, same results bit for bit; ids of
    experts held elsewhere (out of range, negative) are dropped in both."""
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size

    g = torch.Generator().manual_seed(T + E)
    ids = torch.randint(-1, E + 2, (T, k), generator=g)            # int64, some out of range
    a = moe_align_block_size(ids.to(torch.int32).to(dev), block, E, return_counts=True)
    b = moe_align_block_size(ids.to(dev), block, E, return_counts=True)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    rs, re_, rn, rc = og.align_block_size(ids, block, E)
    assert torch.equal(b[3].cpu(), rc.to(torch.int32)) and int(b[2].item()) == int(rn.item())
