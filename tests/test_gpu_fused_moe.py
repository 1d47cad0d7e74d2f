"""GPU parity: fused_moe (bf16/f16, the reference's own operator) and get_start_end vs the CPU
oracle, through the C ABI."""
import pytest
import torch

from oracle import fused_moe as ofm
from oracle import moe_gating as og

pytestmark = pytest.mark.gpu


def _inputs(T, H, I, E, k, seed, dtype, uniform=False):
    g = torch.Generator().manual_seed(seed)
    if uniform:      # the reference fixtures: (rand - 0.5) / 2, test_fused_moe.py:190-205
        mk = lambda *shape: ((torch.rand(shape, generator=g) - 0.5) / 2).to(dtype)
        logits = torch.rand((T, E), generator=g)
    else:
        mk = lambda *shape: (torch.randn(shape, generator=g) * 0.03).to(dtype)
        logits = torch.randn((T, E), generator=g)
    x = mk(T, H) if uniform else torch.randn((T, H), generator=g).to(dtype)
    w1, w2 = mk(E, 2 * I, H), mk(E, H, I)
    tw, ids = og.topk_softmax(logits, k, renormalize=False)
    return x, w1, w2, tw, ids


def test_reference_case(dev):
    # test_fused_moe.py:154-259: seq 128, in 128, hidden 256 (I = 128), out 128, 4 experts, top-2,
    # fp16, renormalize=True, tolerance atol = rtol = 1e-3 (out != in is covered further down)
    from dlcompiler_amd.kernels.fused_moe import fused_moe

    x, w1, w2, tw, ids = _inputs(128, 128, 128, 4, 2, 0, torch.float16, uniform=True)
    out = fused_moe(x.to(dev), w1.to(dev), w2.to(dev), tw.to(dev), ids.to(dev), topk=2,
                    renormalize=True).cpu()
    ref = ofm.fused_moe(x, w1, w2, tw, ids, renormalize=True)
    torch.testing.assert_close(out, ref, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("T,H,I,E,k", [(256, 256, 128, 8, 2), (1, 128, 128, 4, 1),
                                       (333, 512, 384, 64, 6), (512, 2048, 1408, 8, 6)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_moe_parity(dev, T, H, I, E, k, dtype, monkeypatch):
    from dlcompiler_amd.kernels import fused_moe as fm

    x, w1, w2, tw, ids = _inputs(T, H, I, E, k, 1, dtype)
    args = (x.to(dev), w1.to(dev), w2.to(dev), tw.to(dev), ids.to(dev))
    ref = ofm.fused_moe(x, w1, w2, tw, ids, renormalize=True)
    scale = max(1.0, ref.float().abs().max().item())

    def check(out):
        assert out.shape == (T, H) and out.dtype == dtype
        # north-star tolerance for 16-bit outputs: 2e-2 abs/rel, the absolute part taken relative
        # to the output scale (a slot value's 16-bit rounding is proportional to its magnitude)
        torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2 * scale)
        err = ((out.cpu().double() - ref.double()).norm() / ref.double().norm()).item()
        assert err < 5e-3

    check(fm.fused_moe(*args, k, renormalize=True))     # default tile height for row-major weights
    for block in (64, 128):                              # both tile heights, both weight layouts
        monkeypatch.setattr(fm, "_BLOCK_M", block)
        out = fm.fused_moe(*args, k, renormalize=True)
        check(out)
        out2 = fm.fused_moe(args[0], fm.shuffle_moe_weight(args[1]), fm.shuffle_moe_weight(args[2]),
                            args[3], args[4], k, renormalize=True, weights_shuffled=True)
        assert torch.equal(out2, out)


def test_expert_shard(dev):
    from dlcompiler_amd.kernels.fused_moe import fused_moe

    x, w1, w2, tw, ids = _inputs(200, 256, 128, 8, 2, 2, torch.bfloat16)
    d = lambda t: t.to(dev)
    full = fused_moe(d(x), d(w1), d(w2), d(tw), d(ids), 2).cpu().float()
    parts = [fused_moe(d(x), d(w1[o:o + 4].contiguous()), d(w2[o:o + 4].contiguous()), d(tw), d(ids),
                       2, expert_offset=o, num_experts=8).cpu().float() for o in (0, 4)]
    ref = ofm.fused_moe(x, w1[4:], w2[4:], tw, ids, expert_offset=4).float()
    torch.testing.assert_close(parts[1], ref, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(parts[0] + parts[1], full, rtol=2e-2, atol=2e-2)


def test_get_start_end(dev):
    # same values as the reference's docstring identity (fused_moe.py:271-275)
    from dlcompiler_amd.kernels.fused_moe import get_start_end

    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 16, (300, 4), generator=g)
    flat = ids.flatten().to(dev)
    sorted_idx = flat.argsort()
    start, end = get_start_end(flat, sorted_idx, 16)
    rs, re_ = og.start_end(ids, 16)
    assert start.dtype == sorted_idx.dtype
    assert torch.equal(start.cpu(), rs) and torch.equal(end.cpu(), re_)


@pytest.mark.parametrize("out_size", [128, 384])
def test_output_width_comes_from_w2(dev, out_size):
    # the reference sizes the result from w2.shape[1] (fused_moe.py:354-357): it need not be H
    from dlcompiler_amd.kernels.fused_moe import fused_moe

    T, H, I, E, k = 150, 256, 256, 4, 2
    g = torch.Generator().manual_seed(8)
    x = torch.randn((T, H), generator=g).bfloat16()
    tw, ids = og.topk_softmax(torch.randn((T, E), generator=g), k, renormalize=True)
    w1 = (torch.randn((E, 2 * I, H), generator=g) * 0.05).bfloat16()
    w2 = (torch.randn((E, out_size, I), generator=g) * 0.05).bfloat16()
    ref = ofm.fused_moe(x, w1, w2, tw, ids)
    out = fused_moe(x.to(dev), w1.to(dev), w2.to(dev), tw.to(dev), ids.to(dev), k)
    assert out.shape == (T, out_size)
    scale = max(1.0, ref.float().abs().max().item())
    torch.testing.assert_close(out.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2 * scale)


def _launcher_case(dev, M, K, N, E, top_k, dtype, seed=0, enable_weights=True, reindex_a=True,
                   reindex_c=True, idx_dtype=torch.int64, local=None):
    from dlcompiler_amd.kernels.fused_moe import fused_moe_kernel_launcher, get_start_end

    g = torch.Generator().manual_seed(seed)
    A = ((torch.rand((M, K), generator=g) - 0.5) / 2).to(dtype)        # test_fused_moe.py:49-57
    B = ((torch.rand((E, N, K), generator=g) - 0.5) / 2).to(dtype)
    router = torch.rand((M, E), generator=g).to(dtype)
    weights, topk_idx = router.topk(top_k, dim=-1)
    sorted_idx = topk_idx.flatten().argsort(stable=True)                # :9-14
    off, nloc = local if local else (0, E)
    ref = ofm.grouped_gemm_launcher(A, B[off:off + nloc], topk_idx, weights if enable_weights else None,
                                    expert_offset=off)
    ids_d = topk_idx.to(dev)
    exp_start, exp_end = get_start_end(ids_d, sorted_idx.to(idx_dtype).to(dev), E)
    Ad = A.to(dev)
    if not reindex_a:                     # A already holds one row per sorted position
        Ad = A[sorted_idx // top_k].to(dev)
    C = torch.full((M * top_k, N), 7.0, dtype=dtype, device=dev)
    fused_moe_kernel_launcher(Ad, B[off:off + nloc].to(dev), C, sorted_idx.to(idx_dtype).to(dev),
                              exp_start, exp_end, weights.to(dev), enable_weights=enable_weights,
                              top_k=top_k, num_tokens=M, expert_offset=off, reindex_a=reindex_a,
                              reindex_c=reindex_c)
    out = C.cpu()
    if not reindex_c:                     # rows in sorted order -> back to slot order
        back = torch.empty_like(out)
        back[sorted_idx] = out
        out = back
    owned = ((topk_idx >= off) & (topk_idx < off + nloc)).flatten()
    torch.testing.assert_close(out[owned], ref[owned])               # the reference's own tolerance
    assert (out[~owned] == 7.0).all()                                # other experts' rows untouched


def test_reference_launcher_case(dev):
    # test_fused_moe.py:17-145: M 256, K 64, N 128, 4 experts, top-2, fp16, weights enabled
    _launcher_case(dev, 256, 64, 128, 4, 2, torch.float16)


@pytest.mark.parametrize("reindex_a,reindex_c", [(True, False), (False, True), (False, False)])
def test_launcher_reindex_flags(dev, reindex_a, reindex_c):
    # the two calls of fused_moe: gather + sorted rows (fused_moe.py:334-349), sorted + scatter (:358-373)
    _launcher_case(dev, 300, 128, 136, 8, 2, torch.bfloat16, seed=1, reindex_a=reindex_a,
                   reindex_c=reindex_c, enable_weights=reindex_c)


@pytest.mark.parametrize("M,K,N,E,k,dtype,idx", [(1, 64, 8, 2, 1, torch.float16, torch.int32),
                                                 (777, 192, 200, 64, 6, torch.bfloat16, torch.int64),
                                                 (2000, 256, 512, 16, 4, torch.float16, torch.int32),
                                                 (130, 2048, 264, 3, 2, torch.bfloat16, torch.int64)])
def test_launcher_shapes(dev, M, K, N, E, k, dtype, idx):
    _launcher_case(dev, M, K, N, E, k, dtype, seed=M, idx_dtype=idx)
    _launcher_case(dev, M, K, N, E, k, dtype, seed=M + 1, idx_dtype=idx, enable_weights=False)


def test_launcher_expert_shard(dev):
    _launcher_case(dev, 400, 128, 128, 8, 2, torch.float16, seed=3, local=(2, 4))


# sizes that are multiples of 64 but not of 128 (the last gate / up column tile and the last
# output tile are partial), output width a multiple of 8; the reference masks any size
# (fused_moe.py:119-160)
@pytest.mark.parametrize("T,H,I,O,E,k", [(100, 192, 320, 192, 4, 2), (257, 64, 64, 8, 8, 2),
                                         (300, 448, 192, 136, 16, 4)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sizes_that_are_not_multiples_of_128(dev, T, H, I, O, E, k, dtype):
    from dlcompiler_amd.kernels import fused_moe as fm

    g = torch.Generator().manual_seed(T)
    x = torch.randn((T, H), generator=g).to(dtype)
    w1 = (torch.randn((E, 2 * I, H), generator=g) * 0.05).to(dtype)
    w2 = (torch.randn((E, O, I), generator=g) * 0.05).to(dtype)
    tw, ids = og.topk_softmax(torch.randn((T, E), generator=g), k)
    ref = ofm.fused_moe(x, w1, w2, tw, ids)
    out = fm.fused_moe(x.to(dev), w1.to(dev), w2.to(dev), tw.to(dev), ids.to(dev), k).cpu()
    assert out.shape == (T, O)
    scale = max(1.0, ref.float().abs().max().item())
    torch.testing.assert_close(out.float(), ref.float(), rtol=2e-2, atol=2e-2 * scale)
    if O % 16 == 0:   # operand-order weights come in 16-row tiles
        sh = fm.fused_moe(x.to(dev), fm.shuffle_moe_weight(w1.to(dev)), fm.shuffle_moe_weight(w2.to(dev)),
                          tw.to(dev), ids.to(dev), k, weights_shuffled=True).cpu()
        assert torch.equal(sh, out)


def test_operand_order_cache(dev, monkeypatch):
    # row-major weights handed over on every call, re-arranged once on the caller's behalf:
    # same bits as the row-major path, a new copy after an in-place update of the weights
    from dlcompiler_amd.kernels import fused_moe as fm

    x, w1, w2, tw, ids = _inputs(200, 256, 128, 8, 2, 5, torch.bfloat16)
    d = [t.to(dev) for t in (x, w1, w2, tw, ids)]
    plain = fm.fused_moe(*d, 2)
    fm._OPERAND_ORDER_CACHE.clear()
    cached = fm.fused_moe(*d, 2, cache_operand_order=True)
    assert torch.equal(cached, plain) and len(fm._OPERAND_ORDER_CACHE) == 2
    first = fm._OPERAND_ORDER_CACHE[(d[1].data_ptr(), tuple(d[1].shape), d[1].dtype, d[1].device)][1]
    again = fm.fused_moe(*d, 2, cache_operand_order=True)
    assert torch.equal(again, plain)
    assert fm._OPERAND_ORDER_CACHE[(d[1].data_ptr(), tuple(d[1].shape), d[1].dtype, d[1].device)][1] is first
    d[1].mul_(2.0)                                            # in-place update: the copy is stale
    upd = fm.fused_moe(*d, 2, cache_operand_order=True)
    assert torch.equal(upd, fm.fused_moe(*d, 2)) and not torch.equal(upd, plain)
    monkeypatch.setenv("DLBLAS_HIP_CACHE_OPERAND_ORDER", "1")  # the switch for unmodified callers
    assert torch.equal(fm.fused_moe(*d, 2), upd)


def test_zero_tokens(dev):
    """Empty batches (a decode step in which no token is routed to this rank) go through every MoE
    entry point and come back as empty results of the right shape."""
    from dlcompiler_amd.kernels import topk_gating_fwd_part1
    from dlcompiler_amd.kernels.fused_moe import (fused_moe, fused_moe_fp8,
                                                  fused_moe_kernel_launcher)
    from dlcompiler_amd.kernels.moe_gating import moe_topk_softmax_align

    E, H, I, k = 8, 256, 128, 2
    x = torch.empty((0, H), dtype=torch.bfloat16, device=dev)
    w1 = torch.zeros((E, 2 * I, H), dtype=torch.bfloat16, device=dev)
    w2 = torch.zeros((E, H, I), dtype=torch.bfloat16, device=dev)
    tw = torch.empty((0, k), device=dev)
    ids = torch.empty((0, k), dtype=torch.int32, device=dev)
    assert fused_moe(x, w1, w2, tw, ids, k).shape == (0, H)
    w1s = torch.ones((E, 2 * I // 128, H // 128), device=dev)
    w2s = torch.ones((E, H // 128, I // 128), device=dev)
    out = fused_moe_fp8(x, w1.to(torch.float8_e4m3fn), w1s, w2.to(torch.float8_e4m3fn), w2s, tw, ids, k)
    assert out.shape == (0, H) and out.dtype == torch.bfloat16
    gates, masks = topk_gating_fwd_part1.call(torch.empty((0, E), device=dev), k)
    assert gates.shape == (0, E) and masks.shape == (k, 0, E)
    w, i, sorted_ids, expert_ids, npad, counts = moe_topk_softmax_align(
        torch.empty((0, E), device=dev), k, 128, return_counts=True)
    assert w.shape == (0, k) and int(npad.item()) == 0 and (counts == 0).all() and (expert_ids == -1).all()
    C = torch.empty((0, 128), dtype=torch.bfloat16, device=dev)
    none = torch.zeros((4,), dtype=torch.int64, device=dev)
    fused_moe_kernel_launcher(torch.empty((0, 64), dtype=torch.bfloat16, device=dev),
                              torch.zeros((4, 128, 64), dtype=torch.bfloat16, device=dev), C,
                              torch.empty((0,), dtype=torch.int64, device=dev), none, none, None,
                              False, 2, 0, 0, True, True)
    torch.cuda.synchronize()


def test_int64_topk_ids(dev):
    """The ids of torch.topk (int64) go through fused_moe and fused_moe_fp8 unconverted."""
    from dlcompiler_amd.kernels.fused_moe import fused_moe, fused_moe_fp8
    from oracle import fp8 as ofp8

    x, w1, w2, tw, ids = _inputs(200, 256, 128, 8, 2, 21, torch.bfloat16)
    d = [t.to(dev) for t in (x, w1, w2, tw)]
    a = fused_moe(*d, ids.to(dev), topk=2)
    b = fused_moe(*d, ids.long().to(dev), topk=2)
    assert torch.equal(a, b)
    w1q, w1s = ofp8.block_quant_weight(w1.float())
    w2q, w2s = ofp8.block_quant_weight(w2.float())
    q = [t.to(dev) for t in (x, w1q, w1s, w2q, w2s, tw)]
    assert torch.equal(fused_moe_fp8(*q, ids.to(dev), 2), fused_moe_fp8(*q, ids.long().to(dev), 2))
