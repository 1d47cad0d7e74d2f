"""Pins oracle.fp8 / oracle.fused_moe on the CPU: format table, nearest-even brute force,
round-trip bounds, fp64 dense evaluation of the MoE loop."""
import pytest
import torch
import torch.nn.functional as F

from oracle import fp8, fused_moe as ofm, moe_gating as og


def test_decode_table_matches_format_facts_and_torch():
    t = fp8.e4m3fn_decode_table()
    assert t[0x38] == 1.0 and t[0x7E] == 448.0 and t[0x01] == 2.0 ** -9 and t[0x08] == 2.0 ** -6
    assert torch.isnan(t[0x7F]) and torch.isnan(t[0xFF]) and t[0xB8] == -1.0
    via_torch = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).double()
    ok = ~torch.isnan(t)
    assert torch.equal(via_torch[ok], t[ok])


def test_quantiser_is_round_to_nearest_even_bruteforce():
    g = torch.Generator().manual_seed(0)
    x = (torch.randn((64, 256), generator=g) * 3).bfloat16()
    q, s = fp8.per_token_group_quant(x)
    table = fp8.e4m3fn_decode_table()
    finite = table[~torch.isnan(table)]
    y = (x.float().reshape(64, 2, 128) / s[..., None]).reshape(-1).double()
    got = q.float().reshape(-1).double()
    dist = (y[:, None] - finite[None, :]).abs()
    best = dist.min(dim=1).values
    assert torch.equal((y - got).abs(), best)                      # nearest representable
    # ties: exactly two candidates at the same distance -> even mantissa (code) wins
    ties = (dist == best[:, None]).sum(1) > 1
    codes = q.view(torch.uint8).reshape(-1)
    assert (codes[ties] % 2 == 0).all()


def test_quantiser_bounds_saturation_and_zero_groups():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((32, 384), generator=g).bfloat16()
    x[3, 128:256] = 0
    x[5, 7] = 1000.0
    q, s = fp8.per_token_group_quant(x)
    d = fp8.dequant_act(q, s)
    xf = x.float()
    assert s[3, 1].item() == pytest.approx(1e-10 / 448, rel=1e-6) and (d[3, 128:256] == 0).all()
    amax = xf.reshape(32, 3, 128).abs().amax(-1)
    torch.testing.assert_close(s, amax.clamp(min=1e-10) / 448)
    # the group's largest element maps to +-448 exactly
    assert (q.float().reshape(32, 3, 128).abs().amax(-1)[amax > 0] == 448).all()
    # 3 mantissa bits: relative error <= 2^-4 above the subnormal range (|x|/s >= 2^-6)
    normal = (xf.abs() / s.repeat_interleave(128, dim=1)) >= 2.0 ** -6
    rel = ((d - xf).abs() / xf.abs().clamp(min=1e-30))[normal]
    assert rel.max() <= 2.0 ** -4 + 1e-6


def test_weight_block_quant_roundtrip():
    g = torch.Generator().manual_seed(2)
    w = torch.randn((3, 256, 384), generator=g) * 0.02
    q, s = fp8.block_quant_weight(w)
    assert s.shape == (3, 2, 3)
    d = fp8.dequant_weight(q, s)
    blk_amax = w.reshape(3, 2, 128, 3, 128).abs().amax(dim=(2, 4))
    torch.testing.assert_close(s, blk_amax / 448)
    assert ((d - w).abs() <= w.abs() * 2.0 ** -4 + s.repeat_interleave(128, 1).repeat_interleave(128, 2) * 2.0 ** -10).all()


def _moe_inputs(T, H, I, E, k, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, H), generator=g).to(dtype)
    w1 = (torch.randn((E, 2 * I, H), generator=g) * 0.05)
    w2 = (torch.randn((E, H, I), generator=g) * 0.05)
    logits = torch.randn((T, E), generator=g)
    tw, ids = og.topk_softmax(logits, k, renormalize=False)
    return x, w1, w2, tw, ids


def test_bf16_moe_matches_reference_formula_in_fp64():
    # test_fused_moe.py:227-244 evaluated densely in fp64 (routing as a one-hot weight matrix)
    x, w1, w2, tw, ids = _moe_inputs(64, 128, 64, 4, 2, 3)
    w1b, w2b = w1.bfloat16(), w2.bfloat16()
    out = ofm.fused_moe(x, w1b, w2b, tw, ids, renormalize=True)
    wn = (tw / tw.sum(-1, keepdim=True)).double()
    dense = torch.zeros((64, 4), dtype=torch.float64).scatter_(1, ids.long(), wn)
    ref = torch.zeros((64, 128), dtype=torch.float64)
    for e in range(4):
        gate_proj, up_proj = w1b[e].double().chunk(2, dim=0)
        h = F.silu(x.double() @ gate_proj.t()) * (x.double() @ up_proj.t())
        ref += dense[:, e:e + 1] * (h @ w2b[e].double().t())
    torch.testing.assert_close(out.double(), ref, rtol=3e-2, atol=3e-2 * ref.abs().max().item())
    err = (out.double() - ref).norm() / ref.norm()
    assert err < 1e-2


def test_fp8_moe_matches_fp64_dense_evaluation_of_dequantised_operands():
    x, w1, w2, tw, ids = _moe_inputs(48, 256, 128, 4, 2, 4)
    w1q, w1s = fp8.block_quant_weight(w1)
    w2q, w2s = fp8.block_quant_weight(w2)
    out = ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids, renormalize=True)
    xq, xs = fp8.per_token_group_quant(x)
    xd = fp8.dequant_act(xq, xs).double()
    wn = (tw / tw.sum(-1, keepdim=True)).double()
    dense = torch.zeros((48, 4), dtype=torch.float64).scatter_(1, ids.long(), wn)
    ref = torch.zeros((48, 256), dtype=torch.float64)
    for e in range(4):
        w1d = fp8.dequant_weight(w1q[e], w1s[e]).double()
        w2d = fp8.dequant_weight(w2q[e], w2s[e]).double()
        gate_proj, up_proj = w1d.chunk(2, dim=0)
        h = F.silu(xd @ gate_proj.t()) * (xd @ up_proj.t())
        hq, hs = fp8.per_token_group_quant(h.float())
        ref += dense[:, e:e + 1] * (fp8.dequant_act(hq, hs).double() @ w2d.t())
    err = (out.double() - ref).norm() / ref.norm()
    assert err < 1e-2
    # and the quantised pipeline stays close to the unquantised MLP (sanity of the scheme)
    full = ofm.fused_moe(x, w1.bfloat16(), w2.bfloat16(), tw, ids, renormalize=True).double()
    assert (out.double() - full).norm() / full.norm() < 8e-2


def test_expert_offset_selects_a_shard():
    x, w1, w2, tw, ids = _moe_inputs(32, 128, 128, 4, 2, 5)
    w1b, w2b = w1.bfloat16(), w2.bfloat16()
    full = ofm.fused_moe(x, w1b, w2b, tw, ids).float()
    lo = ofm.fused_moe(x, w1b[:2], w2b[:2], tw, ids, expert_offset=0).float()
    hi = ofm.fused_moe(x, w1b[2:], w2b[2:], tw, ids, expert_offset=2).float()
    torch.testing.assert_close(lo + hi, full, rtol=2e-2, atol=2e-2)


def test_grouped_gemm_launcher_is_a_dense_one_hot_product():
    # pins oracle.fused_moe.grouped_gemm_launcher (test_fused_moe.py:97-112) with an fp64 dense
    # evaluation: C[t, j] = sum_e onehot[t, j, e] * (A[t] @ B[e].T) * w[t, j]
    from oracle import fused_moe as ofm

    g = torch.Generator().manual_seed(4)
    M, K, N, E, k = 40, 64, 24, 5, 2
    A = torch.randn((M, K), generator=g)
    B = torch.randn((E, N, K), generator=g)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(M)])
    w = torch.rand((M, k), generator=g)
    got = ofm.grouped_gemm_launcher(A, B, idx, w)
    dense = torch.einsum("mk,enk->men", A.double(), B.double())               # [M, E, N]
    ref = torch.gather(dense, 1, idx[..., None].expand(M, k, N)) * w.double()[..., None]
    torch.testing.assert_close(got.double(), ref.flatten(0, 1), rtol=1e-5, atol=1e-5)
    part = ofm.grouped_gemm_launcher(A, B[2:4], idx, None, expert_offset=2)   # a shard of experts
    mask = ((idx >= 2) & (idx < 4)).flatten()
    full = ofm.grouped_gemm_launcher(A, B, idx, None)
    assert torch.equal(part[mask], full[mask]) and (part[~mask] == 0).all()
