"""GPU parity: paged_attention_fwd, prefill-with-history branch, vs the CPU oracle through the
C ABI."""
import pytest
import torch

from oracle import attention as oa

pytestmark = pytest.mark.gpu


def _run_case(dev, q_lens, hist, hq, hkv, d, page, dtype, seed=0, uniform=False, window=None,
              softcap=None, sm_scale=None, max_seqlen=None, tol=2e-2, dv=None,
              idx_dtypes=(torch.int64,) * 4):
    # idx_dtypes: integer types of (block_offsets, q_start_loc, q_seqlens, kv_seqlens) as handed over
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    gen = torch.Generator().manual_seed(123 + seed)
    if uniform:   # the reference test draws torch.rand inputs (test_paged_attention.py:157-180)
        mk = lambda shape: torch.rand(shape, generator=gen).to(dtype)
    else:
        mk = lambda shape: torch.randn(shape, generator=gen).to(dtype)
    full = [a + b for a, b in zip(q_lens, hist)]
    dv = dv or d
    ks = [mk((max(l, 1), hkv, d))[:l] for l in full]
    vs = [mk((max(l, 1), hkv, dv))[:l] for l in full]
    T = sum(q_lens)
    q = mk((T + 3, hq, d))                                 # 3 rows owned by no sequence
    kc, vc, table = oa.make_paged_cache(ks, vs, page, seed=seed, dtype=dtype)
    start = torch.tensor([sum(q_lens[:i]) for i in range(len(q_lens))])
    ql, kl = torch.tensor(q_lens), torch.tensor(full)
    ref = oa.paged_prefill(q, kc, vc, table, start, ql, kl, sm_scale=sm_scale, window=window,
                           softcap=softcap)
    o = torch.full((T + 3, hq, dv), 9.0, dtype=dtype, device=dev)
    it = idx_dtypes
    ret = paged_attention_fwd(q.to(dev), kc.to(dev), vc.to(dev), o, table.to(it[0]).to(dev),
                              start.to(it[1]).to(dev), ql.to(it[2]).to(dev), kl.to(it[3]).to(dev),
                              max_seqlen or max(q_lens),
                              window_size=window, sm_scale=sm_scale, logit_softcapping=softcap)
    assert ret is None
    out = o.cpu()
    assert (out[T:] == 9.0).all()                         # rows outside every sequence untouched
    assert torch.isfinite(out.float()).all()              # NaN-filled unused cache never read
    torch.testing.assert_close(out[:T].float(), ref[:T].float(), rtol=tol, atol=tol)
    return out[:T], ref[:T]


# the reference's own prefill case (test_paged_attention.py:244-255): seq_lens [30,50,70,90]
# after histories [50,40,30,20], heads (8,2)/(2,2), key head size 48/32 with value head size 32,
# page 16, fp16, uniform inputs -- and the same at the unmasked sizes 64/128
@pytest.mark.parametrize("hq,hkv", [(8, 2), (2, 2)])
@pytest.mark.parametrize("d,dv", [(48, 32), (32, 32), (64, 64), (128, 128)])
def test_reference_prefill_cases(dev, hq, hkv, d, dv):
    out, ref = _run_case(dev, [30, 50, 70, 90], [50, 40, 30, 20], hq, hkv, d, 16, torch.float16,
                         uniform=True, dv=dv)
    torch.testing.assert_close(out.float(), ref.float(), rtol=1e-5, atol=1e-3)


# the reference's window case (test_paged_attention.py:291-303): window 32 on the same lengths
@pytest.mark.parametrize("d,dv", [(48, 32), (64, 64), (128, 128)])
def test_reference_window_case(dev, d, dv):
    out, ref = _run_case(dev, [30, 50, 70, 90], [50, 40, 30, 20], 4, 2, d, 16, torch.float16,
                         uniform=True, window=32, dv=dv)
    torch.testing.assert_close(out.float(), ref.float(), rtol=1e-5, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page", [16, 64, 48])
def test_length_edges(dev, dtype, page):
    # query / history lengths around the 64-key tile, the 128-row block and the page size
    q_lens = [1, 2, 63, 64, 65, 127, 128, 129, 200, 257, 5, 0]
    hist = [0, 63, 1, 64, 127, 0, 128, 300, 77, 1, 1000, 10]
    _run_case(dev, q_lens, hist, 8, 2, 128, page, dtype)


def test_no_history_equals_varlen_prefill(dev):
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    q_lens = [100, 333, 64]
    out, _ = _run_case(dev, q_lens, [0, 0, 0], 8, 2, 128, 64, torch.bfloat16, seed=3)
    gen = torch.Generator().manual_seed(126)
    mk = lambda shape: torch.randn(shape, generator=gen).to(torch.bfloat16)
    ks = [mk((l, 2, 128)) for l in q_lens]
    vs = [mk((l, 2, 128)) for l in q_lens]
    q = mk((sum(q_lens) + 3, 8, 128))[:sum(q_lens)]
    o = torch.empty_like(q, device=dev)
    start = torch.tensor([0, 100, 433], dtype=torch.int32, device=dev)
    context_attention_fwd(q.to(dev), torch.cat(ks).to(dev), torch.cat(vs).to(dev), o, start,
                          torch.tensor(q_lens, dtype=torch.int32, device=dev), max(q_lens))
    assert torch.equal(o.cpu(), out)                      # same kernel body, same tile order


@pytest.mark.parametrize("window", [1, 31, 64, 200, 5000])
def test_sliding_window(dev, window):
    _run_case(dev, [1, 70, 130, 300], [500, 40, 0, 129], 8, 2, 128, 16, torch.bfloat16, window=window)


@pytest.mark.parametrize("softcap", [0.5, 30.0])
def test_logit_softcapping(dev, softcap):
    _run_case(dev, [70, 130, 9], [40, 0, 300], 4, 4, 64, 32, torch.float16, softcap=softcap)


def test_window_and_softcap_and_scale(dev):
    _run_case(dev, [70, 130, 9], [40, 0, 300], 8, 1, 128, 16, torch.bfloat16, softcap=20.0, window=50,
              sm_scale=0.2)


def test_large_chunked_prefill(dev):
    # one 128-row block far into a long context, the chunked-prefill shape
    _run_case(dev, [512, 256], [3000, 1500], 8, 2, 128, 64, torch.bfloat16, seed=5)


# pages that are neither a power of two nor a multiple of a tile: every K/V row is looked up on
# its own, so tiles may straddle pages anywhere
@pytest.mark.parametrize("page", [20, 24, 100])
def test_odd_page_sizes(dev, page):
    _run_case(dev, [70, 33, 129], [45, 0, 200], 4, 2, 128, page, torch.bfloat16, seed=page)
    _run_case(dev, [65], [130], 2, 1, 64, page, torch.float16, seed=page + 1, window=40)


# the prefill branch looks up the page of every K/V row, so any page size works, down to one
# token per page (the decode branch needs multiples of 16)
@pytest.mark.parametrize("page", [1, 4, 8])
def test_small_pages(dev, page):
    _run_case(dev, [70, 33, 129, 1], [45, 0, 200, 7], 4, 2, 128, page, torch.bfloat16, seed=page)
    _run_case(dev, [65, 5], [130, 3], 2, 1, 64, page, torch.float16, seed=page + 1, window=40)


# pages that hold several whole 64-key tiles (a power of two and not): the page of a tile is one
# look-up and the tile starts at a slot that is a multiple of 64 inside it
@pytest.mark.parametrize("page", [128, 192, 256])
def test_pages_of_several_tiles(dev, page):
    _run_case(dev, [70, 33, 129, 1, 300], [45, 0, 200, 700, 1000], 4, 2, 128, page, torch.bfloat16, seed=page)
    _run_case(dev, [65, 130], [130, 500], 2, 1, 64, page, torch.float16, seed=page + 1, window=150)
    _run_case(dev, [64, 128], [64, 256], 8, 2, 128, page, torch.bfloat16, seed=page + 2, softcap=25.0)


# the index tensors are read in the integer width they arrive in: all int32, all int64 (what
# lmdeploy hands over), mixtures, and a narrower type that the wrapper converts
@pytest.mark.parametrize("idx", [(torch.int32,) * 4, (torch.int64,) * 4,
                                 (torch.int64, torch.int32, torch.int64, torch.int32),
                                 (torch.int32, torch.int64, torch.int32, torch.int64),
                                 (torch.int16, torch.int64, torch.int16, torch.int32)])
def test_index_dtypes(dev, idx):
    out = [_run_case(dev, [30, 129, 64], [50, 300, 0], 8, 2, 128, 16, torch.bfloat16, seed=11,
                     idx_dtypes=idx)[0]]
    ref32 = _run_case(dev, [30, 129, 64], [50, 300, 0], 8, 2, 128, 16, torch.bfloat16, seed=11,
                      idx_dtypes=(torch.int32,) * 4)[0]
    assert torch.equal(out[0], ref32)                     # same kernel, same bits


def test_grid_larger_than_needed_and_rejects(dev):
    from dlcompiler_amd import _lib
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    _run_case(dev, [10, 20], [5, 0], 2, 2, 64, 16, torch.float16, max_seqlen=1000)
    q = torch.zeros(8, 2, 100, dtype=torch.float16, device=dev)         # head size not a multiple of 8
    kc = torch.zeros(4, 16, 2, 100, dtype=torch.float16, device=dev)
    with pytest.raises(NotImplementedError):
        paged_attention_fwd(q, kc, kc, torch.empty_like(q), torch.zeros(2, 2, dtype=torch.int32, device=dev),
                            torch.tensor([0, 4], device=dev), torch.tensor([4, 4], device=dev),
                            torch.tensor([4, 4], device=dev), 4)


# the kernel walks the sequences longest context first when the batch fits one workgroup's
# ranking pass (<= 256 sequences) and in index order beyond: both sides of that limit, with
# equal contexts (rank ties) among them
@pytest.mark.parametrize("nseq", [2, 255, 256, 257, 600])
def test_many_sequences_any_order(dev, nseq):
    g = torch.Generator().manual_seed(nseq)
    q_lens = torch.randint(0, 6, (nseq,), generator=g).tolist()
    hist = torch.randint(0, 40, (nseq,), generator=g).tolist()
    hist[1] = hist[0] + q_lens[0] - q_lens[1] if hist[0] + q_lens[0] >= q_lens[1] else hist[1]
    _run_case(dev, q_lens, hist, 4, 2, 128, 16, torch.bfloat16, seed=nseq)


# head sizes that are not powers of two and value sizes that differ from the key size
@pytest.mark.parametrize("d,dv", [(80, 80), (96, 64), (128, 64), (64, 128), (16, 8), (120, 72)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_sizes(dev, d, dv, dtype):
    _run_case(dev, [1, 130, 64, 33], [0, 300, 64, 7], 8, 2, d, 16, dtype, dv=dv, seed=d + dv)
    _run_case(dev, [200], [1000], 4, 4, d, 48, dtype, dv=dv, window=150, softcap=25.0)
