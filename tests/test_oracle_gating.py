"""Pins oracle.moe_gating (CPU): library softmax/top-k, brute force, invariants."""
import itertools

import numpy as np
import pytest
import torch

from oracle import moe_gating as og


def test_topk_matches_torch_topk_of_softmax_on_tie_free_rows():
    g = torch.Generator().manual_seed(1)
    logits = torch.randn((4096, 64), generator=g)
    w, ids = og.topk_softmax(logits, 6, renormalize=False)
    p = torch.softmax(logits, dim=-1, dtype=torch.float32)
    tw, tids = torch.topk(p, 6, dim=-1)           # the reference router, test_fused_moe.py:213-216
    # rows whose top-7 probabilities are all distinct have a unique answer
    top7 = torch.topk(p, 7, dim=-1).values
    unique = (top7[:, :-1] != top7[:, 1:]).all(-1)
    assert unique.float().mean() > 0.99
    assert torch.equal(ids[unique].long(), tids[unique])
    assert torch.equal(w[unique], tw[unique])
    rw, _ = og.topk_softmax(logits, 6, renormalize=True)
    ref = tw / tw.sum(-1, keepdim=True)            # fused_moe.py:322-323
    torch.testing.assert_close(rw[unique], ref[unique], rtol=1e-6, atol=0)
    torch.testing.assert_close(rw.sum(-1), torch.ones(4096), rtol=0, atol=3e-7)


def test_topk_bruteforce_with_crafted_ties():
    logits = torch.tensor([[1.0, 3.0, 3.0, -2.0, 3.0, 0.5, 0.5, 1.0],
                           [0.0, -0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0],
                           [-1.0, -2.0, -3.0, -4.0, -5.0, -6.0, -7.0, -8.0]])
    w, ids = og.topk_softmax(logits, 4, renormalize=True)
    assert ids.tolist() == [[1, 2, 4, 0], [0, 1, 2, 3], [0, 1, 2, 3]]
    for r in range(3):
        row = logits[r].double()
        p = torch.exp(row - row.max())
        p = p / p.sum()
        sel = p[ids[r].long()]
        torch.testing.assert_close(w[r].double(), sel / sel.sum(), rtol=1e-6, atol=0)


def test_topk_invariants_random():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn((512, 160), generator=g)
    w, ids = og.topk_softmax(logits, 8)
    assert (w > 0).all()
    picked = torch.gather(logits, 1, ids.long())
    assert (picked[:, :-1] >= picked[:, 1:]).all()
    assert all(len(set(r)) == 8 for r in ids.tolist())
    # nothing unpicked beats the last picked
    mask = torch.ones_like(logits, dtype=torch.bool).scatter_(1, ids.long(), False)
    assert (logits.masked_fill(~mask, -1e9).max(-1).values <= picked[:, -1]).all()


def test_start_end_is_the_reference_onehot_identity():
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 16, (300, 4), generator=g)
    start, end = og.start_end(ids, 16)
    cnt = torch.nn.functional.one_hot(ids.flatten(), num_classes=16).sum(0)  # fused_moe.py:271-275
    assert torch.equal(end, cnt.cumsum(0))
    assert torch.equal(start, cnt.cumsum(0) - cnt)
    # and it agrees with a stable sort of the flat ids
    order = torch.sort(ids.flatten(), stable=True).indices
    sorted_vals = ids.flatten()[order]
    for e in range(16):
        assert (sorted_vals[start[e]:end[e]] == e).all()


@pytest.mark.parametrize("block,E", [(1, 3), (4, 4), (3, 5), (16, 8)])
def test_align_matches_bruteforce_exhaustively_small(block, E):
    rng = np.random.default_rng(block * 100 + E)
    for n in [0, 1, 2, 7, 33]:
        ids = rng.integers(0, E, size=n).tolist()
        s, e, tot, cnt = og.align_block_size(torch.tensor(ids, dtype=torch.int32).reshape(-1, 1),
                                             block, E)
        bs, be, btot, bcnt = og.align_block_size_bruteforce(ids, block, E)
        assert s.tolist() == bs and e.tolist() == be and tot.item() == btot
        assert cnt.tolist() == bcnt


def test_align_all_assignments_tiny():
    for ids in itertools.product(range(3), repeat=4):
        s, e, tot, cnt = og.align_block_size(torch.tensor(ids, dtype=torch.int32), 2, 3)
        bs, be, btot, bcnt = og.align_block_size_bruteforce(list(ids), 2, 3)
        assert (s.tolist(), e.tolist(), tot.item(), cnt.tolist()) == (bs, be, btot, bcnt)


def check_align_invariants(ids_flat, block, E, s, e, tot, cnt):
    """Size-independent properties of the layout; reused by the GPU tests."""
    ids_flat = np.asarray(ids_flat)
    s, e, cnt = np.asarray(s), np.asarray(e), np.asarray(cnt)
    n = ids_flat.size
    tot = int(tot)
    valid = (ids_flat >= 0) & (ids_flat < E)
    assert cnt.sum() == valid.sum()
    assert tot % block == 0 and tot == (-(-cnt // block) * block).sum()
    real = s[s != n]
    assert np.array_equal(np.sort(real), np.nonzero(valid)[0])       # each slot exactly once
    assert (s[tot:] == n).all() and (e[tot // block:] == -1).all()
    blocks = s[:tot].reshape(-1, block)
    eb = e[:tot // block]
    assert (np.diff(eb) >= 0).all()
    for b in range(blocks.shape[0]):
        row = blocks[b][blocks[b] != n]
        assert (ids_flat[row] == eb[b]).all()
    for x in range(E):
        seg = s[:tot][np.repeat(eb, block) == x]
        seg = seg[seg != n]
        assert (np.diff(seg) > 0).all() and seg.size == cnt[x]


def test_align_invariants_config_size():
    g = torch.Generator().manual_seed(1)
    logits = torch.randn((16384, 64), generator=g)
    _, ids = og.topk_softmax(logits, 6)
    s, e, tot, cnt = og.align_block_size(ids, 64, 64)
    assert s.numel() == 16384 * 6 + 64 * 63
    check_align_invariants(ids.flatten().numpy(), 64, 64, s, e, tot.item(), cnt)


def test_align_drops_out_of_range_ids():
    ids = torch.tensor([0, 5, -1, 1, 9, 1], dtype=torch.int32)
    s, e, tot, cnt = og.align_block_size(ids, 2, 2)
    assert cnt.tolist() == [1, 2] and tot.item() == 4
    assert s.tolist()[:4] == [0, 6, 3, 5]


def test_part1_is_softmax_plus_k_rounds_of_argmax():
    # topk_gating_fwd_part1.py:47-60 against the library routines it is made of
    g = torch.Generator().manual_seed(3)
    logits = torch.randn((2048, 64), generator=g)
    k = 6
    gates, masks = og.topk_gating_part1(logits, k)
    assert gates.shape == (2048, 64) and masks.shape == (k, 2048, 64) and masks.dtype == torch.int64
    p = torch.softmax(logits, dim=-1)
    torch.testing.assert_close(gates, p, rtol=2e-6, atol=0)      # un-shifted vs shifted exponent
    assert (masks.sum(-1) == 1).all()                             # one expert per round
    assert (masks.sum(0) <= 1).all()                              # never the same expert twice
    # rows whose top-(k+1) softmax values are distinct have a unique answer: torch.topk's
    top = torch.topk(p, k + 1, dim=-1)
    unique = (top.values[:, :-1] != top.values[:, 1:]).all(-1)
    gt = torch.topk(gates, k + 1, dim=-1).values
    unique &= (gt[:, :-1] != gt[:, 1:]).all(-1)
    assert unique.float().mean() > 0.99
    picked = masks.argmax(-1).t()                                 # [S, k]
    assert torch.equal(picked[unique], top.indices[unique][:, :k])
    # and the index form of the router says the same
    _, ids = og.topk_softmax(logits, k)
    assert torch.equal(picked[unique], ids[unique].long())


def test_part1_crafted_ties_and_fp16():
    logits = torch.tensor([[1.0, 3.0, 3.0, -2.0, 3.0, 0.5, 0.5, 1.0],
                           [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]])
    gates, masks = og.topk_gating_part1(logits, 4)
    assert masks.argmax(-1).t().tolist() == [[1, 2, 4, 0], [0, 1, 2, 3]]   # lowest index first
    torch.testing.assert_close(gates.sum(-1), torch.ones(2))
    g16, m16 = og.topk_gating_part1(logits.half(), 4)
    assert g16.dtype == torch.float16 and torch.equal(m16, masks)
