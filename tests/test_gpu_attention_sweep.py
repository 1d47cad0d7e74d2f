"""GPU parity: seeded random-shape sweeps of the three attention entry points against the CPU
oracle (ragged lengths around the tile sizes, odd page sizes, GQA ratios, window, soft-cap)."""
import random

import pytest
import torch

from oracle import attention as oa

pytestmark = pytest.mark.gpu

_LENS = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 257]


def _close(out, ref):
    out = out.float()
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out, ref.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("seed", range(24))
def test_prefill_sweep(dev, seed):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    rng = random.Random(100 + seed)
    d = rng.choice([64, 128])
    hkv = rng.choice([1, 2, 4])
    hq = hkv * rng.choice([1, 2, 4])
    dtype = rng.choice([torch.bfloat16, torch.float16])
    nseq = rng.randint(1, 4)
    lens = [rng.choice(_LENS + [rng.randint(1, 700)]) for _ in range(nseq)]
    gen = torch.Generator().manual_seed(1000 + seed)
    T = sum(lens)
    q = torch.randn((T, hq, d), generator=gen).to(dtype)
    k = torch.randn((T, hkv, d), generator=gen).to(dtype)
    v = torch.randn((T, hkv, d), generator=gen).to(dtype)
    start = torch.tensor([sum(lens[:i]) for i in range(nseq)], dtype=torch.int32)
    sl = torch.tensor(lens, dtype=torch.int32)
    o = torch.zeros_like(q, device=dev)
    context_attention_fwd(q.to(dev), k.to(dev), v.to(dev), o, start.to(dev), sl.to(dev), max(lens))
    _close(o.cpu(), oa.prefill_attention(q, k, v, start, sl))

    # the same queries after a history, through the paged cache
    page = rng.choice([16, 20, 32, 48, 64, 128])
    if T == nseq:
        page = rng.choice([16, 32, 64])  # one token per sequence takes the decode branch
    hist = [rng.choice([0, 1, 17, 64, 100, rng.randint(0, 500)]) for _ in range(nseq)]
    full = [a + b for a, b in zip(lens, hist)]
    ks = [torch.randn((n, hkv, d), generator=gen).to(dtype) for n in full]
    vs = [torch.randn((n, hkv, d), generator=gen).to(dtype) for n in full]
    kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=seed, dtype=dtype)
    window = rng.choice([None, None, 16, 100])
    softcap = rng.choice([None, None, 30.0])
    ql, kl = torch.tensor(lens), torch.tensor(full)
    o2 = torch.zeros_like(q, device=dev)
    paged_attention_fwd(q.to(dev), kc.to(dev), vc.to(dev), o2, table.to(dev), start.to(dev),
                        ql.to(dev), kl.to(dev), max(lens), window_size=window,
                        logit_softcapping=softcap)
    _close(o2.cpu(), oa.paged_prefill(q, kc, vc, table, start.long(), ql, kl, window=window,
                                      softcap=softcap))


@pytest.mark.parametrize("seed", range(24))
def test_decode_sweep(dev, seed):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    rng = random.Random(200 + seed)
    d = rng.choice([64, 128])
    hkv = rng.choice([1, 2, 8])
    hq = hkv * rng.choice([1, 4, 8, 16])
    dtype = rng.choice([torch.bfloat16, torch.float16])
    B = rng.choice([1, 2, 5, 17, 64])
    page = rng.choice([16, 32, 48, 64, 128])
    ctx = [rng.choice([1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 129, 500, rng.randint(1, 3000)])
           for _ in range(B)]
    gen = torch.Generator().manual_seed(2000 + seed)
    ks = [torch.randn((n, hkv, d), generator=gen).to(dtype) for n in ctx]
    vs = [torch.randn((n, hkv, d), generator=gen).to(dtype) for n in ctx]
    kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=seed, dtype=dtype)
    q = torch.randn((B, hq, d), generator=gen).to(dtype)
    window = rng.choice([None, None, 16, 100])
    softcap = rng.choice([None, None, 30.0])
    kl = torch.tensor(ctx)
    o = torch.zeros_like(q, device=dev)
    paged_attention_fwd(q.to(dev), kc.to(dev), vc.to(dev), o, table.to(dev),
                        torch.arange(B, device=dev), torch.ones(B, dtype=torch.int64, device=dev),
                        kl.to(dev), 1, window_size=window, logit_softcapping=softcap)
    _close(o.cpu(), oa.paged_decode(q, kc, vc, table, kl, window=window, softcap=softcap))


# head sizes that are any multiple of 8 (key and value size drawn independently), all three paths
@pytest.mark.parametrize("seed", range(16))
def test_head_size_sweep(dev, seed):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    rng = random.Random(300 + seed)
    d = 8 * rng.randint(1, 16)
    dv = rng.choice([d, 8 * rng.randint(1, 16)])
    hkv = rng.choice([1, 2])
    hq = hkv * rng.choice([1, 4])
    dtype = rng.choice([torch.bfloat16, torch.float16])
    gen = torch.Generator().manual_seed(3000 + seed)
    nseq = rng.randint(1, 3)
    lens = [rng.choice(_LENS) for _ in range(nseq)]
    T = sum(lens)
    start = torch.tensor([sum(lens[:i]) for i in range(nseq)], dtype=torch.int32)
    sl = torch.tensor(lens, dtype=torch.int32)
    q = torch.randn((T, hq, d), generator=gen).to(dtype)

    # packed prefill (one head size for q, k and v)
    k = torch.randn((T, hkv, d), generator=gen).to(dtype)
    v = torch.randn((T, hkv, d), generator=gen).to(dtype)
    o = torch.zeros_like(q, device=dev)
    context_attention_fwd(q.to(dev), k.to(dev), v.to(dev), o, start.to(dev), sl.to(dev), max(lens))
    _close(o.cpu(), oa.prefill_attention(q, k, v, start, sl))

    # paged prefill after a history and paged decode, value size dv
    page = rng.choice([16, 32, 64])
    hist = [rng.choice([0, 17, 100]) for _ in range(nseq)]
    full = [a + b for a, b in zip(lens, hist)]
    ks = [torch.randn((n, hkv, d), generator=gen).to(dtype) for n in full]
    vs = [torch.randn((n, hkv, dv), generator=gen).to(dtype) for n in full]
    kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=seed, dtype=dtype)
    ql, kl = torch.tensor(lens), torch.tensor(full)
    if T != nseq:
        o2 = torch.zeros((T, hq, dv), dtype=dtype, device=dev)
        paged_attention_fwd(q.to(dev), kc.to(dev), vc.to(dev), o2, table.to(dev), start.to(dev),
                            ql.to(dev), kl.to(dev), max(lens))
        _close(o2.cpu(), oa.paged_prefill(q, kc, vc, table, start.long(), ql, kl))
    qd = torch.randn((nseq, hq, d), generator=gen).to(dtype)
    o3 = torch.zeros((nseq, hq, dv), dtype=dtype, device=dev)
    paged_attention_fwd(qd.to(dev), kc.to(dev), vc.to(dev), o3, table.to(dev),
                        torch.arange(nseq, device=dev), torch.ones(nseq, dtype=torch.int64, device=dev),
                        kl.to(dev), 1)
    _close(o3.cpu(), oa.paged_decode(qd, kc, vc, table, kl))


# head sizes above 128 (up to 256: one kernel instance, one wavefront per SIMD), e.g. the 192 / 128
# of a multi-head-latent prefill and the 256 of some dense models; all three paths
@pytest.mark.parametrize("d,dv", [(256, 256), (192, 128), (136, 136), (160, 256), (248, 8), (64, 192),
                                  (256, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_large_head_sizes(dev, d, dv, dtype):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    seed = d * 3 + dv
    rng = random.Random(seed)
    hkv = rng.choice([1, 2])
    hq = hkv * rng.choice([1, 4])
    gen = torch.Generator().manual_seed(seed)
    lens = [rng.choice([1, 63, 64, 65, 130, 257]) for _ in range(3)]
    nseq, T = len(lens), sum(lens)
    start = torch.tensor([sum(lens[:i]) for i in range(nseq)], dtype=torch.int32)
    sl = torch.tensor(lens, dtype=torch.int32)
    q = torch.randn((T, hq, d), generator=gen).to(dtype)
    k = torch.randn((T, hkv, d), generator=gen).to(dtype)
    v = torch.randn((T, hkv, d), generator=gen).to(dtype)
    o = torch.zeros_like(q, device=dev)
    context_attention_fwd(q.to(dev), k.to(dev), v.to(dev), o, start.to(dev), sl.to(dev), max(lens))
    _close(o.cpu(), oa.prefill_attention(q, k, v, start, sl))

    for page in (16, 64, 48):
        hist = [rng.choice([0, 17, 100, 300]) for _ in range(nseq)]
        full = [a + b for a, b in zip(lens, hist)]
        ks = [torch.randn((n, hkv, d), generator=gen).to(dtype) for n in full]
        vs = [torch.randn((n, hkv, dv), generator=gen).to(dtype) for n in full]
        kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=seed, dtype=dtype)
        ql, kl = torch.tensor(lens), torch.tensor(full)
        o2 = torch.zeros((T, hq, dv), dtype=dtype, device=dev)
        paged_attention_fwd(q.to(dev), kc.to(dev), vc.to(dev), o2, table.to(dev), start.to(dev),
                            ql.to(dev), kl.to(dev), max(lens))
        _close(o2.cpu(), oa.paged_prefill(q, kc, vc, table, start.long(), ql, kl))
        qd = torch.randn((nseq, hq, d), generator=gen).to(dtype)
        o3 = torch.zeros((nseq, hq, dv), dtype=dtype, device=dev)
        window = rng.choice([None, 50])
        paged_attention_fwd(qd.to(dev), kc.to(dev), vc.to(dev), o3, table.to(dev),
                            torch.arange(nseq, device=dev), torch.ones(nseq, dtype=torch.int64, device=dev),
                            kl.to(dev), 1, window_size=window)
        _close(o3.cpu(), oa.paged_decode(qd, kc, vc, table, kl, window=window))


def test_config_size_attention_repeats_bit_identically(dev):
    """Config-size prefill and paged decode, repeated: both kernels copy K/V into LDS with
    hand-issued loads and explicit waits; a missing wait would show as run-to-run differences."""
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    g = torch.Generator().manual_seed(21)
    Hq, Hkv, D, page = 32, 8, 128, 64
    lens = torch.randint(512, 4097, (8,), generator=g, dtype=torch.int32)
    start = (torch.cumsum(lens, 0, dtype=torch.int32) - lens).to(dev)
    total = int(lens.sum())
    q = torch.randn((total, Hq, D), generator=g).bfloat16().to(dev)
    k = torch.randn((total, Hkv, D), generator=g).bfloat16().to(dev)
    v = torch.randn((total, Hkv, D), generator=g).bfloat16().to(dev)
    o = torch.empty_like(q)
    lens_d = lens.to(dev)
    context_attention_fwd(q, k, v, o, start, lens_d, int(lens.max()))
    first = o.clone()
    assert torch.isfinite(first.float()).all()
    for _ in range(5):
        o.zero_()
        context_attention_fwd(q, k, v, o, start, lens_d, int(lens.max()))
        assert torch.equal(o, first)

    B = 64
    ctx = torch.randint(512, 8193, (B,), generator=g, dtype=torch.int32)
    pages_per = 8192 // page
    npages = B * pages_per
    kc = torch.randn((npages, page, Hkv, D), generator=g).bfloat16().to(dev)
    vc = torch.randn((npages, page, Hkv, D), generator=g).bfloat16().to(dev)
    bt = torch.randperm(npages, generator=g).to(torch.int32).view(B, pages_per).to(dev)
    qd = torch.randn((B, Hq, D), generator=g).bfloat16().to(dev)
    od = torch.empty_like(qd)
    qsl = torch.arange(B, dtype=torch.int32).to(dev)
    qlen = torch.ones(B, dtype=torch.int32).to(dev)
    ctx_d = ctx.to(dev)
    paged_attention_fwd(qd, kc, vc, od, bt, qsl, qlen, ctx_d, 1)
    firstd = od.clone()
    assert torch.isfinite(firstd.float()).all()
    for _ in range(5):
        od.zero_()
        paged_attention_fwd(qd, kc, vc, od, bt, qsl, qlen, ctx_d, 1)
        assert torch.equal(od, firstd)
