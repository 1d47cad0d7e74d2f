"""GPU parity: fp8 quantiser and fp8 fused MoE vs the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import fp8 as ofp8
from oracle import fused_moe as ofm
from oracle import moe_gating as og

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(4096, 2048), (1, 128), (77, 1408), (300, 384)])
def test_quant_is_bit_exact(dev, dtype, shape):
    from dlcompiler_amd.kernels.fused_moe import per_token_group_quant_fp8

    g = torch.Generator().manual_seed(0)
    x = (torch.randn(shape, generator=g) * 2).to(dtype)
    if shape[0] > 3:
        x[1, :128] = 0                      # zero group -> eps scale
        x[2, 5] = 3000.0                    # outlier
        x[3, :] = x[3, :].abs().clamp(min=1e-3) * 1e-6   # tiny values
    q, s = per_token_group_quant_fp8(x.to(dev))
    rq, rs = ofp8.per_token_group_quant(x)
    assert torch.equal(s.cpu(), rs)
    assert torch.equal(q.cpu().view(torch.uint8), rq.view(torch.uint8))


def _inputs(T, H, I, E, k, seed, dtype=torch.bfloat16, wstd=0.02):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, H), generator=g).to(dtype)
    logits = torch.randn((T, E), generator=g)
    w1 = torch.randn((E, 2 * I, H), generator=g) * wstd
    w2 = torch.randn((E, H, I), generator=g) * wstd
    tw, ids = og.topk_softmax(logits, k, renormalize=True)
    w1q, w1s = ofp8.block_quant_weight(w1)
    w2q, w2s = ofp8.block_quant_weight(w2)
    return x, w1q, w1s, w2q, w2s, tw, ids


def _rel_err(out, ref):
    return ((out.double() - ref.double()).norm() / ref.double().norm()).item()


def _check(out, ref):
    # north-star: <= 3e-2 relative against the dequantised fp32 GEMM
    assert _rel_err(out, ref) <= 3e-2
    scale = ref.float().abs().max().item()
    torch.testing.assert_close(out.float(), ref.float(), rtol=3e-2, atol=3e-2 * scale)


@pytest.mark.parametrize("T,H,I,E,k", [(128, 256, 128, 4, 2), (512, 2048, 1408, 8, 6),
                                       (1, 256, 256, 8, 2), (333, 512, 384, 64, 6),
                                       (64, 128, 128, 2, 1),
                                       # K of 4096 / 2304 bytes: more than one 16-chunk window of scales
                                       (96, 4096, 2304, 4, 2)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_moe_fp8_parity(dev, T, H, I, E, k, dtype, monkeypatch):
    from dlcompiler_amd.kernels import fused_moe as fm

    x, w1q, w1s, w2q, w2s, tw, ids = _inputs(T, H, I, E, k, 1, dtype)
    ref = ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids)
    d = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s, tw, ids)]
    out = fm.fused_moe_fp8(*d, k)
    assert out.shape == (T, H) and out.dtype == dtype
    _check(out.cpu(), ref)
    sh = fm.shuffle_moe_weight_fp8
    for block in (64, 128):                      # both tile heights, both weight layouts
        monkeypatch.setattr(fm, "_BLOCK_M", block)
        plain = fm.fused_moe_fp8(*d, k)
        _check(plain.cpu(), ref)
        # operand-order weight storage: same bytes re-arranged, so the result is bit-identical
        shuf = fm.fused_moe_fp8(d[0], sh(d[1]), d[2], sh(d[3]), d[4], d[5], d[6], k,
                                weights_shuffled=True)
        assert torch.equal(shuf, plain)


def test_weight_shuffle_layout(dev):
    # the documented address formula of the operand-order layout, checked element by element
    from dlcompiler_amd.kernels.fused_moe import shuffle_moe_weight_fp8

    E, N, K = 2, 32, 256
    w = torch.arange(E * N * K, dtype=torch.int64).remainder(251).to(torch.uint8)
    w = w.view(E, N, K)
    sh = shuffle_moe_weight_fp8(w.view(torch.float8_e4m3fn).to(dev)).cpu().view(torch.uint8).flatten()
    for e, nb, kc, h, l, b in [(0, 0, 0, 0, 0, 0), (1, 1, 1, 1, 63, 15), (0, 1, 0, 1, 17, 3),
                               (1, 0, 1, 0, 40, 9)]:
        addr = ((e * (N // 16) + nb) * (K // 128) + kc) * 2048 + h * 1024 + l * 16 + b
        assert sh[addr] == w[e, 16 * nb + l % 16, 128 * kc + 64 * h + 16 * (l // 16) + b]


def test_one_hot_routing_reduces_to_a_single_expert_mlp(dev):
    from dlcompiler_amd.kernels.fused_moe import fused_moe_fp8

    x, w1q, w1s, w2q, w2s, _, _ = _inputs(200, 256, 256, 4, 1, 2)
    ids = torch.full((200, 1), 2, dtype=torch.int32)
    tw = torch.ones((200, 1))
    out = fused_moe_fp8(x.to(dev), w1q.to(dev), w1s.to(dev), w2q.to(dev), w2s.to(dev),
                        tw.to(dev), ids.to(dev), 1).cpu()
    xd = ofp8.dequant_act(*ofp8.per_token_group_quant(x))
    h = xd @ ofp8.dequant_weight(w1q[2], w1s[2]).t()
    gate, up = h.chunk(2, -1)
    act = torch.nn.functional.silu(gate) * up
    ad = ofp8.dequant_act(*ofp8.per_token_group_quant(act))
    ref = (ad @ ofp8.dequant_weight(w2q[2], w2s[2]).t()).bfloat16()
    _check(out, ref)


def test_renormalize_and_linearity_in_routing_weight(dev):
    from dlcompiler_amd.kernels.fused_moe import fused_moe_fp8

    x, w1q, w1s, w2q, w2s, tw, ids = _inputs(256, 256, 128, 8, 2, 3)
    args = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s)]
    base = fused_moe_fp8(*args, tw.to(dev), ids.to(dev), 2).cpu()
    # renormalize=True on weights scaled by a constant gives the same result
    ren = fused_moe_fp8(*args, (tw * 3).to(dev), ids.to(dev), 2, renormalize=True).cpu()
    torch.testing.assert_close(ren.float(), base.float(), rtol=2e-2, atol=1e-3)
    # doubling the routing weights doubles every slot output before the top-k sum
    dbl = fused_moe_fp8(*args, (tw * 2).to(dev), ids.to(dev), 2).cpu()
    torch.testing.assert_close(dbl.float(), base.float() * 2, rtol=1.6e-2, atol=1e-3)


def test_expert_sharding_adds_up(dev):
    from dlcompiler_amd.kernels.fused_moe import fused_moe_fp8

    x, w1q, w1s, w2q, w2s, tw, ids = _inputs(300, 256, 128, 8, 2, 4)
    d = lambda t: t.to(dev)
    full = fused_moe_fp8(d(x), d(w1q), d(w1s), d(w2q), d(w2s), d(tw), d(ids), 2).cpu().float()
    parts = []
    for off in (0, 4):
        sl = slice(off, off + 4)
        parts.append(fused_moe_fp8(d(x), d(w1q[sl].contiguous()), d(w1s[sl].contiguous()),
                                   d(w2q[sl].contiguous()), d(w2s[sl].contiguous()), d(tw), d(ids),
                                   2, expert_offset=off, num_experts=8).cpu().float())
        ref = ofm.fused_moe_fp8(x, w1q[sl], w1s[sl], w2q[sl], w2s[sl], tw, ids, expert_offset=off)
        _check(parts[-1], ref)
    torch.testing.assert_close(parts[0] + parts[1], full, rtol=2e-2, atol=2e-2 * full.abs().max().item())


def test_deterministic(dev):
    from dlcompiler_amd.kernels.fused_moe import fused_moe_fp8

    x, w1q, w1s, w2q, w2s, tw, ids = _inputs(512, 512, 256, 16, 4, 5)
    args = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s, tw, ids)]
    a = fused_moe_fp8(*args, 4)
    b = fused_moe_fp8(*args, 4)
    assert torch.equal(a, b)


def test_config5_full(dev):
    """benchmark configuration 5: 4096 tokens, hidden 2048, intermediate 1408, 64 experts, top-6."""
    from dlcompiler_amd.kernels.fused_moe import fused_moe_fp8

    T, H, I, E, k = 4096, 2048, 1408, 64, 6
    g = torch.Generator().manual_seed(5)
    x = torch.randn((T, H), generator=g).bfloat16()
    logits = torch.randn((T, E), generator=g)
    tw, ids = og.topk_softmax(logits, k)
    w1q = torch.empty((E, 2 * I, H), dtype=torch.float8_e4m3fn)
    w1s = torch.empty((E, 2 * I // 128, H // 128))
    w2q = torch.empty((E, H, I), dtype=torch.float8_e4m3fn)
    w2s = torch.empty((E, H // 128, I // 128))
    for e in range(E):                               # quantise expert by expert (memory)
        w1q[e], w1s[e] = ofp8.block_quant_weight(torch.randn((2 * I, H), generator=g) * 0.02)
        w2q[e], w2s[e] = ofp8.block_quant_weight(torch.randn((H, I), generator=g) * 0.02)
    from dlcompiler_amd.kernels.fused_moe import shuffle_moe_weight_fp8

    out = fused_moe_fp8(x.to(dev), shuffle_moe_weight_fp8(w1q.to(dev)), w1s.to(dev),
                        shuffle_moe_weight_fp8(w2q.to(dev)), w2s.to(dev), tw.to(dev), ids.to(dev),
                        k, weights_shuffled=True).cpu()
    assert torch.isfinite(out.float()).all()
    # oracle on a token sample: tokens are independent given the weights
    pick = torch.arange(0, T, 37)
    ref = ofm.fused_moe_fp8(x[pick], w1q, w1s, w2q, w2s, tw[pick], ids[pick])
    _check(out[pick], ref)


@pytest.mark.parametrize("block", [64, 128])
def test_fused_moe_fp8_repeats_bit_identically(dev, block, monkeypatch):
    """Config-size run, repeated: the kernel issues its LDS copies by hand with explicit waits, so
    a missing wait would show as run-to-run differences on a busy chip."""
    from dlcompiler_amd.kernels import fused_moe as fm

    T, H, I, E, k = 4096, 2048, 1408, 64, 6
    g = torch.Generator().manual_seed(9)
    x = torch.randn((T, H), generator=g).bfloat16().to(dev)
    w1q = (torch.randn((E, 2 * I, H), generator=g) * 0.5).to(torch.float8_e4m3fn).to(dev)
    w2q = (torch.randn((E, H, I), generator=g) * 0.5).to(torch.float8_e4m3fn).to(dev)
    w1s = (torch.rand((E, 2 * I // 128, H // 128), generator=g) * 0.02 + 0.01).to(dev)
    w2s = (torch.rand((E, H // 128, I // 128), generator=g) * 0.02 + 0.01).to(dev)
    tw, ids = torch.topk(torch.softmax(torch.randn((T, E), generator=g), -1), k)
    tw, ids = tw.to(dev), ids.int().to(dev)
    monkeypatch.setattr(fm, "_BLOCK_M", block)
    for shuffled in (False, True):
        a = fm.shuffle_moe_weight_fp8(w1q) if shuffled else w1q
        b = fm.shuffle_moe_weight_fp8(w2q) if shuffled else w2q
        first = fm.fused_moe_fp8(x, a, w1s, b, w2s, tw, ids, k, weights_shuffled=shuffled).clone()
        assert torch.isfinite(first.float()).all()
        for _ in range(8):
            again = fm.fused_moe_fp8(x, a, w1s, b, w2s, tw, ids, k, weights_shuffled=shuffled)
            assert torch.equal(again, first)
    # both weight layouts hold the same numbers: same result
    plain = fm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids, k, weights_shuffled=False)
    assert torch.equal(plain, first)


@pytest.mark.parametrize("out_size", [128, 384])
def test_output_width_comes_from_w2(dev, out_size):
    # the reference sizes the result from w2.shape[1] (fused_moe.py:354-357): it need not be H
    from dlcompiler_amd.kernels.fused_moe import fused_moe_fp8

    T, H, I, E, k = 150, 256, 256, 4, 2
    g = torch.Generator().manual_seed(7)
    x = torch.randn((T, H), generator=g).bfloat16()
    tw, ids = og.topk_softmax(torch.randn((T, E), generator=g), k, renormalize=True)
    w1q, w1s = ofp8.block_quant_weight(torch.randn((E, 2 * I, H), generator=g) * 0.05)
    w2q, w2s = ofp8.block_quant_weight(torch.randn((E, out_size, I), generator=g) * 0.05)
    ref = ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids)
    out = fused_moe_fp8(*[t.to(dev) for t in (x, w1q, w1s, w2q, w2s, tw, ids)], k)
    assert out.shape == (T, out_size)
    _check(out.cpu(), ref)


# The GEMM keeps its accumulators relative to the scale of the current 128-deep chunk and moves
# them from chunk to chunk with the ratio of neighbouring scales: rows whose neighbouring groups
# differ by many orders of magnitude are the cases in which that ratio is extreme.  Every case is
# checked against the dequantised fp32 evaluation at the usual tolerance and must stay finite.
@pytest.mark.parametrize("case", ["zero_groups", "outlier_group", "tiny_activations",
                                  "block_scale_spread", "scale_floor", "zero_weight_blocks"])
def test_dynamic_range(dev, case):
    from dlcompiler_amd.kernels import fused_moe as fm

    T, H, I, E, k = 192, 1024, 512, 4, 2
    g = torch.Generator().manual_seed(17)
    x = torch.randn((T, H), generator=g)
    w1 = torch.randn((E, 2 * I, H), generator=g) * 0.05
    w2 = torch.randn((E, H, I), generator=g) * 0.05
    tw, ids = og.topk_softmax(torch.randn((T, E), generator=g), k, renormalize=True)
    if case == "zero_groups":            # all-zero 128-groups between normal ones, and a zero row
        x[::2, 128:256] = 0
        x[::3, 512:768] = 0
        x[1::4, 896:] = 0                # zero tail: the LAST chunk's scale is the eps scale
        x[5] = 0
    elif case == "outlier_group":        # one group 3000 x larger than its neighbours
        x[:, 256:384] *= 3000.0
        x[7, 0:128] *= 1e-4
    elif case == "tiny_activations":     # an intermediate below the quantiser's eps (1e-10): its
        x *= 1e-5                        # groups all carry the floor scale; some input groups too
        x[::2, 384:512] *= 1e-7
    x = x.to(torch.bfloat16)
    w1q, w1s = ofp8.block_quant_weight(w1)
    w2q, w2s = ofp8.block_quant_weight(w2)
    if case == "block_scale_spread":     # block scales from 1e-6 to 1e+2 inside one expert
        f = 10.0 ** torch.linspace(-6, 2, w1s[0].numel()).reshape(w1s[0].shape)
        w1s = w1s * f[None] * 1e-3 / w1s.mean()
        f2 = 10.0 ** torch.linspace(2, -6, w2s[0].numel()).reshape(w2s[0].shape)
        w2s = w2s * f2[None] * 1e-3 / w2s.mean()
    elif case == "scale_floor":          # block scales far below anything the kernel keeps apart
        w1s[:, :, 2] = 1e-30
        w1s[:, 1, :] = 1e-30
        w2s[:, :, 1] = 1e-30
    elif case == "zero_weight_blocks":   # all-zero weight blocks quantised with the scale 0
        w1q8 = w1q.view(torch.uint8)
        w1q8[:, 128:256, 256:384] = 0
        w1q8[:, :, 896:] = 0             # the last chunk of every row
        w1s[:, 1, 2] = 0.0
        w1s[:, :, 7] = 0.0
        w2q.view(torch.uint8)[:, 256:384, :128] = 0
        w2s[:, 2, 0] = 0.0
    ref = ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids)
    assert torch.isfinite(ref.float()).all()
    d = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s, tw, ids)]
    for shuffled in (False, True):
        if shuffled:
            d[1], d[3] = fm.shuffle_moe_weight_fp8(d[1]), fm.shuffle_moe_weight_fp8(d[3])
        out = fm.fused_moe_fp8(*d, k, weights_shuffled=shuffled).cpu()
        assert torch.isfinite(out.float()).all()
        assert _rel_err(out, ref) <= 3e-2, (case, _rel_err(out, ref))


# alignment + quantisation as one native call (the quantiser rides in the placement launch) gives
# what the two separate operators give, bit for bit, across the chunk-size regimes of the alignment
@pytest.mark.parametrize("T,H,E,k", [(4096, 2048, 64, 6), (1, 128, 8, 2), (77, 384, 60, 6),
                                     (16384, 256, 64, 6), (300, 1408, 256, 8), (90000, 128, 16, 6)])
def test_align_and_quant_one_call(dev, T, H, E, k):
    from dlcompiler_amd.kernels import fused_moe as fm
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size

    g = torch.Generator().manual_seed(T + E)
    x = (torch.randn((T, H), generator=g) * 3).to(torch.bfloat16).to(dev)
    ids = torch.randint(0, E, (T, k), generator=g).to(torch.int32).to(dev)
    sorted_ids, counts, xq, xs = fm._align_and_quant(ids, fm.ALIGN_BLOCK, E, x)
    rs, _, rn, rc = moe_align_block_size(ids, fm.ALIGN_BLOCK, E, return_counts=True)
    rq, rsc = fm.per_token_group_quant_fp8(x)
    assert torch.equal(sorted_ids, rs) and torch.equal(counts, rc)
    assert torch.equal(xq.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(xs, rsc)
    os_, _, _, oc = og.align_block_size(ids.cpu(), fm.ALIGN_BLOCK, E)
    npad = int(rn.item())
    assert torch.equal(sorted_ids.cpu()[:npad], os_[:npad]) and torch.equal(counts.cpu(), oc)


# a caller that already holds the alignment of its routing (from the router call) hands it over:
# same result bit for bit as when fused_moe_fp8 / fused_moe sort the routing themselves
def test_alignment_handed_over(dev):
    from dlcompiler_amd.kernels import fused_moe as fm
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size, moe_topk_softmax_align

    T, H, I, E, k = 320, 512, 256, 16, 4
    g = torch.Generator().manual_seed(31)
    x = torch.randn((T, H), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    w1 = torch.randn((E, 2 * I, H), generator=g) * 0.05
    w2 = torch.randn((E, H, I), generator=g) * 0.05
    w1q, w1s = ofp8.block_quant_weight(w1)
    w2q, w2s = ofp8.block_quant_weight(w2)
    tw, ids, sorted_ids, _, _, counts = moe_topk_softmax_align(logits.to(dev), k, fm.ALIGN_BLOCK,
                                                               return_counts=True)
    rw, rids = og.topk_softmax(logits, k)
    assert torch.equal(ids.cpu(), rids)
    assert torch.equal(counts.cpu(), og.expert_counts(rids, E))
    d = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s)]
    base = fm.fused_moe_fp8(*d, tw, ids, k)
    handed = fm.fused_moe_fp8(*d, tw, ids, k, alignment=(sorted_ids, counts))
    assert torch.equal(base, handed)
    _check(base.cpu(), ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, rw, rids))
    s2, _, _, c2 = moe_align_block_size(ids, fm.ALIGN_BLOCK, E, return_counts=True)
    b16 = fm.fused_moe(d[0], w1.to(torch.bfloat16).to(dev), w2.to(torch.bfloat16).to(dev), tw, ids, k)
    h16 = fm.fused_moe(d[0], w1.to(torch.bfloat16).to(dev), w2.to(torch.bfloat16).to(dev), tw, ids, k,
                       alignment=(s2, c2))
    assert torch.equal(b16, h16)
    with pytest.raises(ValueError):      # an alignment built with another block size does not fit
        s64, _, _, c64 = moe_align_block_size(ids, 8, E, return_counts=True)
        fm.fused_moe_fp8(*d, tw, ids, k, alignment=(s64, c64))
