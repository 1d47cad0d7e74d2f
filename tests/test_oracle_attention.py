"""Pins oracle.attention (CPU) against torch's SDPA and closed-form cases."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attention as oa


def _rand(shape, seed, dtype=torch.bfloat16):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


@pytest.mark.parametrize("hq,hkv", [(6, 6), (8, 2), (4, 1)])
def test_prefill_matches_sdpa(hq, hkv):
    lens = [5, 64, 1, 33]
    total = sum(lens)
    q, k, v = _rand((total, hq, 32), 0), _rand((total, hkv, 32), 1), _rand((total, hkv, 32), 2)
    start = torch.tensor([0, 5, 69, 70], dtype=torch.int32)
    o = oa.prefill_attention(q, k, v, start, torch.tensor(lens, dtype=torch.int32))
    for s, l in zip(start.tolist(), lens):
        ref = F.scaled_dot_product_attention(
            q[s:s + l].float().transpose(0, 1)[None], k[s:s + l].float().transpose(0, 1)[None],
            v[s:s + l].float().transpose(0, 1)[None], is_causal=True, enable_gqa=True)[0]
        # only difference: the oracle rounds P to bf16 before P.V (as the reference does)
        torch.testing.assert_close(o[s:s + l].float(), ref.transpose(0, 1), rtol=2e-2, atol=2e-2)


def test_prefill_fp32_is_exactly_sdpa_semantics():
    q, k, v = (_rand((40, 4, 16), i, torch.float32) for i in range(3))
    o = oa.prefill_attention(q, k, v, torch.tensor([0, 17]), torch.tensor([17, 23]))
    for s, l in [(0, 17), (17, 23)]:
        ref = F.scaled_dot_product_attention(q[s:s + l].transpose(0, 1)[None],
                                             k[s:s + l].transpose(0, 1)[None],
                                             v[s:s + l].transpose(0, 1)[None], is_causal=True)[0]
        torch.testing.assert_close(o[s:s + l], ref.transpose(0, 1), rtol=1e-5, atol=1e-6)


def test_prefill_closed_forms():
    # first token of every sequence attends only to itself -> output = its V row
    q, k, v = _rand((12, 4, 16), 0), _rand((12, 2, 16), 1), _rand((12, 2, 16), 2)
    o = oa.prefill_attention(q, k, v, torch.tensor([0, 7]), torch.tensor([7, 5]))
    for s in (0, 7):
        assert torch.equal(o[s], v[s].repeat_interleave(2, dim=0))
    # identical keys -> uniform probabilities -> causal prefix mean of V
    k2 = k[:1].expand(12, 2, 16).contiguous()
    o2 = oa.prefill_attention(q, k2, v, torch.tensor([0]), torch.tensor([12]))
    prefix = v.float().cumsum(0) / torch.arange(1, 13)[:, None, None]
    torch.testing.assert_close(o2.float(), prefix.repeat_interleave(2, dim=1), rtol=2e-2, atol=2e-2)
    # GQA mapping: query head h uses kv head h // group
    v3 = torch.zeros_like(v)
    v3[:, 1] = 1.0
    o3 = oa.prefill_attention(q, k, v3, torch.tensor([0]), torch.tensor([12]))
    assert (o3[:, :2] == 0).all() and (o3[:, 2:] == 1).all()


def test_paged_decode_matches_dense_and_is_permutation_invariant():
    lens = [1, 64, 65, 130, 17]
    ks = [_rand((l, 2, 32), 10 + i) for i, l in enumerate(lens)]
    vs = [_rand((l, 2, 32), 20 + i) for i, l in enumerate(lens)]
    q = _rand((5, 8, 32), 3)
    outs = []
    for seed in (0, 1):
        kc, vc, table = oa.make_paged_cache(ks, vs, page=16, num_pages=40, seed=seed)
        outs.append(oa.paged_decode(q, kc, vc, table, torch.tensor(lens)))
    assert torch.equal(outs[0], outs[1])                  # page placement does not matter
    for b, l in enumerate(lens):
        ref = F.scaled_dot_product_attention(q[b].float()[None, :, None, :],
                                             ks[b].float().transpose(0, 1)[None],
                                             vs[b].float().transpose(0, 1)[None],
                                             enable_gqa=True)[0, :, 0]
        torch.testing.assert_close(outs[0][b].float(), ref, rtol=2e-2, atol=2e-2)
    assert torch.equal(outs[0][0], vs[0][0].repeat_interleave(4, dim=0))   # ctx = 1


def test_paged_decode_zero_length_and_scale():
    ks, vs = [_rand((20, 1, 16), 1)], [_rand((20, 1, 16), 2)]
    kc, vc, table = oa.make_paged_cache(ks, vs, page=16)
    q = _rand((1, 2, 16), 3)
    assert (oa.paged_decode(q, kc, vc, table, torch.tensor([0])) == 0).all()
    a = oa.paged_decode(q, kc, vc, table, torch.tensor([20]), sm_scale=0.0)
    torch.testing.assert_close(a[0, 0].float(), vs[0][:, 0].float().mean(0), rtol=2e-2, atol=2e-2)
    assert math.isfinite(a.float().sum().item())


def test_window_and_softcap_closed_forms():
    ks, vs = [_rand((50, 1, 16), 1)], [_rand((50, 1, 16), 2)]
    kc, vc, table = oa.make_paged_cache(ks, vs, page=16)
    q = _rand((1, 2, 16), 3)
    n = torch.tensor([50])
    base = oa.paged_decode(q, kc, vc, table, n)
    assert torch.equal(oa.paged_decode(q, kc, vc, table, n, window=49), base)      # window covers all
    assert torch.equal(oa.paged_decode(q, kc, vc, table, n, window=1000), base)
    # the window keeps the current token and `window` older ones: same as a shorter context
    short = oa.make_paged_cache([ks[0][39:]], [vs[0][39:]], page=16)
    assert torch.equal(oa.paged_decode(q, kc, vc, table, n, window=10),
                       oa.paged_decode(q, short[0], short[1], short[2], torch.tensor([11])))
    # soft cap: huge cap is the identity, tiny cap flattens the logits -> mean of V
    torch.testing.assert_close(oa.paged_decode(q, kc, vc, table, n, softcap=1e6).float(), base.float(),
                               rtol=1e-2, atol=1e-2)
    flat = oa.paged_decode(q, kc, vc, table, n, softcap=1e-4)
    torch.testing.assert_close(flat[0, 0].float(), vs[0][:, 0].float().mean(0), rtol=2e-2, atol=2e-2)


def _paged_prefill_case(q_lens, hist, hq=4, hkv=2, d=16, page=16, seed=0):
    full = [a + b for a, b in zip(q_lens, hist)]
    ks = [_rand((l, hkv, d), 10 + i) for i, l in enumerate(full)]
    vs = [_rand((l, hkv, d), 20 + i) for i, l in enumerate(full)]
    q = _rand((sum(q_lens), hq, d), 3)
    kc, vc, table = oa.make_paged_cache(ks, vs, page=page, seed=seed)
    start = torch.tensor([sum(q_lens[:i]) for i in range(len(q_lens))])
    return q, ks, vs, kc, vc, table, start, torch.tensor(q_lens), torch.tensor(full)


def test_paged_prefill_reduces_to_prefill_and_decode():
    q_lens, hist = [30, 50, 7, 1], [50, 0, 30, 20]
    q, ks, vs, kc, vc, table, start, ql, kl = _paged_prefill_case(q_lens, hist)
    out = oa.paged_prefill(q, kc, vc, table, start, ql, kl)
    # no history: packed varlen prefill of the same tokens
    ref1 = oa.prefill_attention(q[30:80], ks[1], vs[1], torch.tensor([0]), torch.tensor([50]))
    assert torch.equal(out[30:80], ref1)
    # every query row alone is a decode step over the context that ends at its position
    for b in range(4):
        for i in (0, q_lens[b] - 1):
            ctx = hist[b] + i + 1
            row = oa.paged_decode(q[start[b] + i][None], kc, vc, table[b][None], torch.tensor([ctx]))
            assert torch.equal(out[start[b] + i], row[0])
    # additive-bias formulation of the reference test (key j hidden when j - i > history)
    b = 0
    kk = ks[b].float().repeat_interleave(2, dim=1).permute(1, 2, 0)            # [Hq, D, Lk]
    vv = vs[b].float().repeat_interleave(2, dim=1).transpose(0, 1)             # [Hq, Lk, D]
    qq = q[:30].float().transpose(0, 1)                                        # [Hq, Lq, D]
    i = torch.arange(30)[:, None]
    j = torch.arange(80)[None, :]
    bias = ((j - i) > hist[b]).float() * -1e30
    p = torch.softmax(qq @ kk / math.sqrt(16) + bias, dim=-1).to(q.dtype).float()
    torch.testing.assert_close(out[:30].float(), (p @ vv).transpose(0, 1), rtol=2e-2, atol=2e-2)


def test_paged_prefill_window():
    q_lens, hist = [30, 12], [50, 40]
    q, ks, vs, kc, vc, table, start, ql, kl = _paged_prefill_case(q_lens, hist)
    base = oa.paged_prefill(q, kc, vc, table, start, ql, kl)
    assert torch.equal(oa.paged_prefill(q, kc, vc, table, start, ql, kl, window=1000), base)
    out = oa.paged_prefill(q, kc, vc, table, start, ql, kl, window=8)
    # each row: decode over the context ending at its position with the same window
    for b in range(2):
        for i in range(q_lens[b]):
            ctx = hist[b] + i + 1
            row = oa.paged_decode(q[start[b] + i][None], kc, vc, table[b][None], torch.tensor([ctx]),
                                  window=8)
            assert torch.equal(out[start[b] + i], row[0])


def test_value_head_size_may_differ_from_key_head_size():
    # the reference's own paged-attention matrix runs key size 48 / 32 with value size 32
    # (test_paged_attention.py:244-246); pinned here by torch's SDPA on the gathered context
    g = torch.Generator().manual_seed(21)
    lens = [37, 5, 64]
    hq, hkv, dk, dv, page = 4, 2, 48, 32, 16
    ks = [torch.randn((l, hkv, dk), generator=g) for l in lens]
    vs = [torch.randn((l, hkv, dv), generator=g) for l in lens]
    q = torch.randn((len(lens), hq, dk), generator=g)
    kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=1)
    assert kc.shape[-1] == dk and vc.shape[-1] == dv
    out = oa.paged_decode(q, kc, vc, table, torch.tensor(lens))
    assert out.shape == (len(lens), hq, dv)
    for b, l in enumerate(lens):
        kk = ks[b].transpose(0, 1).repeat_interleave(hq // hkv, 0)
        vv = vs[b].transpose(0, 1).repeat_interleave(hq // hkv, 0)
        ref = torch.nn.functional.scaled_dot_product_attention(q[b][:, None, :], kk, vv)[:, 0]
        torch.testing.assert_close(out[b], ref, rtol=1e-5, atol=1e-5)
    # prefill with history: every query row equals a decode over the context ending at it
    q_lens, hist = [7, 3], [11, 0]
    full = [a + b for a, b in zip(q_lens, hist)]
    ks = [torch.randn((l, hkv, dk), generator=g) for l in full]
    vs = [torch.randn((l, hkv, dv), generator=g) for l in full]
    kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=2)
    qp = torch.randn((sum(q_lens), hq, dk), generator=g)
    start = torch.tensor([0, q_lens[0]])
    o = oa.paged_prefill(qp, kc, vc, table, start, torch.tensor(q_lens), torch.tensor(full))
    assert o.shape == (sum(q_lens), hq, dv)
    for b in range(2):
        for i in range(q_lens[b]):
            row = start[b].item() + i
            one = oa.paged_decode(qp[row][None], kc, vc, table[b][None], torch.tensor([hist[b] + i + 1]))
            torch.testing.assert_close(o[row], one[0], rtol=1e-5, atol=1e-5)
