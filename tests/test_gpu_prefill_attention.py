"""GPU parity: context_attention_fwd vs the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import attention as oa

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype, mean=0.0, std=1.0):
    x = torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * std + mean
    return x.to(dtype)


def _run(dev, lens, hq, hkv, d, dtype, stats=((0, 1), (0, 1), (0, 1)), gap=0, atol=2e-2, rtol=2e-2,
         idx_dtypes=(torch.int32, torch.int32)):
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    starts, at = [], 0
    for l in lens:
        starts.append(at)
        at += l + gap                       # optional unused rows between sequences
    total = max(at, 1)
    q = _rand((total, hq, d), 0, dtype, *stats[0])
    k = _rand((total, hkv, d), 1, dtype, *stats[1])
    v = _rand((total, hkv, d), 2, dtype, *stats[2])
    start = torch.tensor(starts, dtype=torch.int32)
    seqlen = torch.tensor(lens, dtype=torch.int32)
    ref = oa.prefill_attention(q, k, v, start, seqlen)
    o = torch.full((total, hq, d), 5.0, dtype=dtype, device=dev)
    ret = context_attention_fwd(q.to(dev), k.to(dev), v.to(dev), o, start.to(idx_dtypes[0]).to(dev),
                                seqlen.to(idx_dtypes[1]).to(dev), max(lens) if lens else 0)
    assert ret is None
    out = o.cpu()
    inside = torch.zeros(total, dtype=torch.bool)
    for s, l in zip(starts, lens):
        inside[s:s + l] = True
    torch.testing.assert_close(out[inside].float(), ref[inside].float(), rtol=rtol, atol=atol)
    assert (out[~inside] == 5.0).all()      # rows outside every sequence are untouched
    return out, ref


def test_reference_case(dev):
    # test_prefill_attention.py:38-83: 4 sequences {512, 1024, 512, 1024}, 6 heads (MHA),
    # head_dim 128, fp16, q ~ N(.1,.2), k ~ N(.4,.2), v ~ N(.3,.2); tolerance atol 1e-2, rtol 0
    _run(dev, [512, 1024, 512, 1024], 6, 6, 128, torch.float16,
         stats=((0.1, 0.2), (0.4, 0.2), (0.3, 0.2)), atol=1e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128])
def test_length_edges_gqa(dev, dtype, d):
    lens = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257, 700]
    _run(dev, lens, 8, 2, d, dtype)


# b_start_loc / b_seq_len are read in the integer width they arrive in
@pytest.mark.parametrize("idx", [(torch.int64, torch.int64), (torch.int32, torch.int64),
                                 (torch.int64, torch.int32), (torch.int16, torch.uint8)])
def test_index_dtypes(dev, idx):
    lens = [5, 130, 64, 200]
    out, _ = _run(dev, lens, 8, 2, 128, torch.bfloat16, gap=3, idx_dtypes=idx)
    ref32, _ = _run(dev, lens, 8, 2, 128, torch.bfloat16, gap=3)
    assert torch.equal(out, ref32)


def test_group_sizes(dev):
    for hq, hkv in [(4, 4), (8, 1), (32, 8), (12, 4), (3, 1)]:
        _run(dev, [300, 17, 130], hq, hkv, 128, torch.bfloat16)


def test_gaps_empty_sequences_and_single(dev):
    _run(dev, [100, 0, 260, 1], 8, 2, 128, torch.bfloat16, gap=3)
    _run(dev, [1], 8, 8, 64, torch.float16)


def test_closed_forms(dev):
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    dt = torch.bfloat16
    L = 300
    q = _rand((L, 8, 128), 0, dt).to(dev)
    v = _rand((L, 2, 128), 2, dt)
    k = _rand((1, 2, 128), 1, dt).expand(L, 2, 128).contiguous().to(dev)   # identical keys
    o = torch.empty_like(q)
    start = torch.tensor([0], dtype=torch.int32, device=dev)
    lens = torch.tensor([L], dtype=torch.int32, device=dev)
    context_attention_fwd(q, k, v.to(dev), o, start, lens, L)
    prefix = v.float().cumsum(0) / torch.arange(1, L + 1)[:, None, None]
    torch.testing.assert_close(o.cpu().float(), prefix.repeat_interleave(4, dim=1),
                               rtol=2e-2, atol=2e-2)
    assert torch.equal(o[0].cpu(), v[0].repeat_interleave(4, dim=0))        # row 0 = V[0]


def test_strided_qkv_views(dev):
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    dt = torch.bfloat16
    L, hq, hkv, d = 200, 8, 2, 128
    qkv = _rand((L, hq + 2 * hkv, d), 3, dt)
    qkv_d = qkv.to(dev)
    q, k, v = qkv_d[:, :hq], qkv_d[:, hq:hq + hkv], qkv_d[:, hq + hkv:]
    o = torch.empty((L, hq, d), dtype=dt, device=dev)
    context_attention_fwd(q, k, v, o, torch.tensor([0, 120], device=dev),
                          torch.tensor([120, 80], device=dev), 120)
    ref = oa.prefill_attention(qkv[:, :hq].contiguous(), qkv[:, hq:hq + hkv].contiguous(),
                               qkv[:, hq + hkv:].contiguous(), torch.tensor([0, 120]),
                               torch.tensor([120, 80]))
    torch.testing.assert_close(o.cpu().float(), ref.float(), rtol=2e-2, atol=2e-2)


def test_config3_full(dev):
    """benchmark configuration 3: 8 sequences with lengths uniform in [512, 4096] (seed 2), 32 query /
    8 KV heads, head_dim 128, bf16 ~ N(0,1)."""
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    g = torch.Generator().manual_seed(2)
    lens = torch.randint(512, 4097, (8,), generator=g)
    cu = torch.zeros(9, dtype=torch.int32)
    cu[1:] = lens.cumsum(0)
    total = int(cu[-1])
    q = torch.randn((total, 32, 128), generator=g).bfloat16()
    k = torch.randn((total, 8, 128), generator=g).bfloat16()
    v = torch.randn((total, 8, 128), generator=g).bfloat16()
    o = torch.empty((total, 32, 128), dtype=torch.bfloat16, device=dev)
    context_attention_fwd(q.to(dev), k.to(dev), v.to(dev), o, cu[:-1].to(dev),
                          (cu[1:] - cu[:-1]).to(dev), int(lens.max()))
    out = o.cpu()
    assert torch.isfinite(out.float()).all()
    # oracle on the shortest sequence in full and on 4 heads (one per KV group pair) of the
    # longest; sequences and heads are independent
    i_min, i_max = int(lens.argmin()), int(lens.argmax())
    s, l = int(cu[i_min]), int(lens[i_min])
    ref = oa.prefill_attention(q[s:s + l], k[s:s + l], v[s:s + l], torch.tensor([0]), torch.tensor([l]))
    torch.testing.assert_close(out[s:s + l].float(), ref.float(), rtol=2e-2, atol=2e-2)
    s, l = int(cu[i_max]), int(lens[i_max])
    heads = [0, 9, 18, 31]
    for h in heads:
        ref = oa.prefill_attention(q[s:s + l, h:h + 1], k[s:s + l, h // 4:h // 4 + 1],
                                   v[s:s + l, h // 4:h // 4 + 1], torch.tensor([0]), torch.tensor([l]))
        torch.testing.assert_close(out[s:s + l, h:h + 1].float(), ref.float(), rtol=2e-2, atol=2e-2)
    # every first token of a sequence must reproduce its own V row exactly
    for b in range(8):
        assert torch.equal(out[int(cu[b])], v[int(cu[b])].repeat_interleave(4, dim=0))


# the head sizes the reference's wrapper accepts (prefill_attention.py:160: 16, 32, 64, 128) and
# sizes in between; 64 and 128 run the unmasked kernels, the others the masked variants
@pytest.mark.parametrize("d", [16, 32, 48, 80, 96, 120])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_head_sizes(dev, d, dtype):
    _run(dev, [1, 33, 64, 129, 700], 8, 2, d, dtype, gap=2)


# the exponent reference of a row is set by its first tile and only moves up by steps larger
# than 8: scores far below zero, far above it, and a late key that dwarfs everything before it
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_score_ranges(dev, dtype):
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    L, hq, hkv, d = 300, 4, 2, 128
    g = torch.Generator().manual_seed(11)
    q = torch.randn((L, hq, d), generator=g)
    k = torch.randn((L, hkv, d), generator=g)
    v = torch.randn((L, hkv, d), generator=g).to(dtype)
    start, seqlen = torch.tensor([0], dtype=torch.int32), torch.tensor([L], dtype=torch.int32)
    cases = {
        "large negative scores": (q * 6, -q[:, :hkv].abs().mean(0, keepdim=True).expand(L, hkv, d) * 6 + k * 0.1),
        "large positive scores": (q.abs() * 4, k.abs() * 4),
        "late dominant key": (q, torch.cat([k[:200] * 0.05, k[200:201] * 0 + q[250, :hkv] * 3, k[201:] * 0.05])),
    }
    for name, (qq, kk) in cases.items():
        qq, kk = qq.to(dtype), kk.to(dtype)
        ref = oa.prefill_attention(qq, kk, v, start, seqlen)
        o = torch.empty((L, hq, d), dtype=dtype, device=dev)
        context_attention_fwd(qq.to(dev), kk.to(dev), v.to(dev), o, start.to(dev), seqlen.to(dev), L)
        out = o.cpu().float()
        assert torch.isfinite(out).all(), name
        torch.testing.assert_close(out, ref.float(), rtol=2e-2, atol=2e-2, msg=lambda m: f"{name}: {m}")
