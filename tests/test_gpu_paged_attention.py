"""GPU parity: paged_attention_fwd (decode branch) vs the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import attention as oa

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


def _run_case(dev, lens, hq, hkv, d, page, dtype, seed=0, num_pages=None, table_dtype=torch.int32,
              sm_scale=None, uniform=False, window=None, softcap=None, dv=None, len_dtype=torch.int64):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    if uniform:   # the reference test draws torch.rand inputs (test_paged_attention.py:157-180)
        gen = torch.Generator().manual_seed(123)
        mk = lambda shape, s: torch.rand(shape, generator=gen).to(dtype)
    else:
        mk = lambda shape, s: _rand(shape, s, dtype)
    B = len(lens)
    dv = dv or d
    ks = [mk((max(l, 1), hkv, d), 100 + i)[:l] for i, l in enumerate(lens)]
    vs = [mk((max(l, 1), hkv, dv), 200 + i)[:l] for i, l in enumerate(lens)]
    q = mk((B, hq, d), 7)
    kc, vc, table = oa.make_paged_cache(ks, vs, page, num_pages=num_pages, seed=seed, dtype=dtype)
    kv_len = torch.tensor(lens)
    ref = oa.paged_decode(q, kc, vc, table, kv_len, sm_scale=sm_scale, window=window, softcap=softcap)
    o = torch.full((B, hq, dv), 9.0, dtype=dtype, device=dev)
    ret = paged_attention_fwd(q.to(dev), kc.to(dev), vc.to(dev), o, table.to(table_dtype).to(dev),
                              torch.arange(B, device=dev), torch.ones(B, dtype=torch.int64, device=dev),
                              kv_len.to(len_dtype).to(dev), 1, sm_scale=sm_scale, window_size=window,
                              logit_softcapping=softcap)
    assert ret is None
    out = o.cpu()
    assert torch.isfinite(out.float()).all()              # NaN-filled unused cache never read
    # north-star tolerance for 16-bit outputs: 2e-2 abs/rel
    torch.testing.assert_close(out.float(), ref.float(), rtol=2e-2, atol=2e-2)
    return out, ref


# the reference's own cases (test_paged_attention.py:244-255): decode rows seq_lens [1,1,1,1],
# history [50,40,30,20], heads (8,2)/(2,2), key head size 48/32 with value head size 32, page 16,
# fp16, uniform inputs -- and the same at the unmasked sizes 64/128
@pytest.mark.parametrize("hq,hkv", [(8, 2), (2, 2)])
@pytest.mark.parametrize("d,dv", [(48, 32), (32, 32), (64, 64), (128, 128)])
def test_reference_decode_cases(dev, hq, hkv, d, dv):
    out, ref = _run_case(dev, [51, 41, 31, 21], hq, hkv, d, 16, torch.float16, uniform=True,
                         table_dtype=torch.int64, dv=dv)
    # the reference's tolerance is atol 1e-3 on values in [0, 1]
    torch.testing.assert_close(out.float(), ref.float(), rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page", [16, 64, 128])
def test_context_length_edges(dev, dtype, page):
    lens = [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 511, 512, 513, 1000, 0]
    _run_case(dev, lens, 32, 8, 128, page, dtype)


# block table and context lengths are read in the integer width they arrive in
@pytest.mark.parametrize("table_dtype,len_dtype", [(torch.int32, torch.int32), (torch.int64, torch.int64),
                                                   (torch.int32, torch.int64), (torch.int64, torch.int32),
                                                   (torch.int16, torch.int16)])
def test_index_dtypes(dev, table_dtype, len_dtype):
    lens = [1, 17, 300, 1025, 64, 0, 2049]
    out, _ = _run_case(dev, lens, 32, 8, 128, 16, torch.bfloat16, table_dtype=table_dtype,
                       len_dtype=len_dtype)
    ref32, _ = _run_case(dev, lens, 32, 8, 128, 16, torch.bfloat16)
    assert torch.equal(out, ref32)
    _run_case(dev, [513, 77], 8, 2, 64, 48, torch.float16, table_dtype=table_dtype, len_dtype=len_dtype)


def test_group_sizes_and_scale(dev):
    for hq, hkv in [(8, 8), (16, 2), (32, 1), (40, 2)]:
        _run_case(dev, [300, 77, 1025], hq, hkv, 64, 32, torch.bfloat16, sm_scale=0.2)


# the reference's window case uses win_size 32 on the same sequences (test_paged_attention.py:
# 288-346, ground truth from flash_attn which is not available here; the oracle restates the
# kernel's own mask, paged_attention.py:163-167,191-199)
@pytest.mark.parametrize("window", [32, 1, 600, 5000])
def test_sliding_window(dev, window):
    _run_case(dev, [51, 41, 31, 21, 1, 700, 2049], 8, 2, 128, 16, torch.float16, window=window)
    _run_case(dev, [513, 1200, 64], 32, 8, 128, 64, torch.bfloat16, window=window)


@pytest.mark.parametrize("cap", [30.0, 5.0, 0.5])
def test_logit_softcapping(dev, cap):
    _run_case(dev, [300, 77, 1025, 1], 16, 4, 128, 64, torch.bfloat16, softcap=cap)
    _run_case(dev, [300, 2000], 8, 2, 64, 16, torch.float16, softcap=cap, window=100)


def test_many_short_sequences(dev):
    # more sequences than lanes in a wavefront and contexts far shorter than a work piece: a
    # piece then spans many sequences and the per-sequence scan walks several blocks of 64
    gen = torch.Generator().manual_seed(11)
    lens = torch.randint(0, 70, (150,), generator=gen).tolist()
    lens[0], lens[64], lens[149] = 1, 0, 33
    _run_case(dev, lens, 8, 2, 128, 16, torch.bfloat16, seed=4)
    _run_case(dev, lens[:131], 4, 4, 64, 32, torch.float16, seed=5, window=20)


def test_one_long_sequence_many_pieces(dev):
    # a single long context is cut into many pieces (one partial each)
    _run_case(dev, [20000], 8, 2, 128, 64, torch.bfloat16, seed=6)
    _run_case(dev, [3, 20000, 5], 8, 8, 64, 16, torch.float16, seed=7, window=3000)


def test_non_power_of_two_page_and_spare_pages(dev):
    _run_case(dev, [700, 48, 49, 1], 8, 2, 128, 48, torch.bfloat16, num_pages=64)


def test_page_placement_invariance(dev):
    a, _ = _run_case(dev, [900, 130, 64], 32, 8, 128, 64, torch.bfloat16, seed=0, num_pages=40)
    b, _ = _run_case(dev, [900, 130, 64], 32, 8, 128, 64, torch.bfloat16, seed=5, num_pages=40)
    assert torch.equal(a, b)


def test_strided_views(dev):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    dtype = torch.bfloat16
    lens = [200, 90]
    ks = [_rand((l, 2, 64), 1 + i, dtype) for i, l in enumerate(lens)]
    vs = [_rand((l, 2, 64), 5 + i, dtype) for i, l in enumerate(lens)]
    kc, vc, table = oa.make_paged_cache(ks, vs, 16)
    # K and V interleaved in one allocation: [pages, page, 2, H, D] -> strided views
    kv = torch.stack([kc, vc], dim=2).to(dev)
    qkv = _rand((2, 8 + 4, 64), 9, dtype).to(dev)
    q = qkv[:, :8]                                          # row stride 12*64
    o = torch.zeros((2, 8, 64), dtype=dtype, device=dev)
    paged_attention_fwd(q, kv[:, :, 0], kv[:, :, 1], o, table.to(dev), None,
                        torch.ones(2, device=dev), torch.tensor(lens, device=dev), 1)
    ref = oa.paged_decode(q.cpu().contiguous(), kc, vc, table, torch.tensor(lens))
    torch.testing.assert_close(o.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)


def test_unsupported_requests_raise(dev):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    def args(d):
        q = torch.zeros((2, 4, d), dtype=torch.float16, device=dev)
        kc = torch.zeros((4, 16, 2, d), dtype=torch.float16, device=dev)
        return (q, kc, kc, torch.zeros_like(q), torch.zeros((2, 2), dtype=torch.int32, device=dev),
                None, torch.ones(2, device=dev), torch.tensor([3, 4], device=dev), 1)

    with pytest.raises(NotImplementedError):
        paged_attention_fwd(*args(44))                       # head size not a multiple of 8
    with pytest.raises(NotImplementedError):
        paged_attention_fwd(*args(264))                      # head size above 256
    q = torch.zeros((2, 4, 64), dtype=torch.float16, device=dev)
    kc = torch.zeros((4, 8, 2, 64), dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):                 # decode pages are multiples of 16
        paged_attention_fwd(q, kc, kc, torch.zeros_like(q), torch.zeros((2, 2), dtype=torch.int32, device=dev),
                            None, torch.ones(2, device=dev), torch.tensor([3, 4], device=dev), 1)


def test_config4_full(dev):
    """benchmark configuration 4: batch 64, ctx uniform in [512, 8192] (seed 3), 64-token pages,
    32 query / 8 KV heads, head_dim 128, bf16; block table [64, 128] from a seeded permutation."""
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    g = torch.Generator().manual_seed(3)
    ctx = torch.randint(512, 8193, (64,), generator=g)
    blocks = (ctx + 63) // 64
    num_pages = int(blocks.sum())
    perm = torch.randperm(num_pages, generator=g).to(torch.int32)
    table = torch.zeros((64, 128), dtype=torch.int32)
    at = 0
    for b in range(64):
        table[b, :blocks[b]] = perm[at:at + blocks[b]]
        at += int(blocks[b])
    kc = torch.randn((num_pages, 64, 8, 128), generator=g).bfloat16()
    vc = torch.randn((num_pages, 64, 8, 128), generator=g).bfloat16()
    q = torch.randn((64, 32, 128), generator=g).bfloat16()
    o = torch.empty((64, 32, 128), dtype=torch.bfloat16, device=dev)
    kcd, vcd = kc.to(dev), vc.to(dev)
    paged_attention_fwd(q.to(dev), kcd, vcd, o, table.to(dev), None, torch.ones(64, device=dev),
                        ctx.to(dev), 1)
    out = o.cpu()
    # oracle on a sample of sequences incl. the shortest and longest (each is independent)
    pick = sorted({int(ctx.argmin()), int(ctx.argmax()), 0, 17, 40, 63})
    ref = oa.paged_decode(q[pick], kc, vc, table[pick], ctx[pick])
    torch.testing.assert_close(out[pick].float(), ref.float(), rtol=2e-2, atol=2e-2)
    # whole-batch property: the output is a convex combination of V rows
    assert torch.isfinite(out.float()).all()
    assert out.float().abs().max() <= vc.float().abs().max()


# head sizes that are not powers of two and value sizes that differ from the key size (the
# reference splits them into power-of-two blocks, paged_attention.py:531-539)
@pytest.mark.parametrize("d,dv", [(80, 80), (96, 96), (96, 64), (128, 64), (64, 128), (16, 8),
                                  (120, 72), (40, 104)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_sizes(dev, d, dv, dtype):
    _run_case(dev, [1, 17, 300, 1025, 64], 8, 2, d, 16, dtype, dv=dv, seed=d + dv)
    _run_case(dev, [700, 33], 4, 4, d, 64, dtype, dv=dv, window=100, softcap=20.0)
