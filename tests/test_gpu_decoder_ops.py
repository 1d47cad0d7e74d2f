"""GPU parity: fill_kv_cache, rms_norm / add_rms_norm, apply_rotary_pos_emb vs the CPU oracle."""
import pytest
import torch

from oracle import decoder_ops as od

pytestmark = pytest.mark.gpu


def _div_up(a, b):
    return (a + b - 1) // b


# cases of the reference test (test_fill_kv_cache.py:139-146): 8 heads, head_dim 128, page 64
@pytest.mark.parametrize("seq_lens,history_lens", [((1, 1, 1, 1), (1, 16, 31, 24)),
                                                   ((1, 8, 16, 24), (1, 16, 31, 24)),
                                                   ((70, 1, 130), (0, 63, 64))])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("idx", [torch.int64, torch.int32, "mixed"])
def test_fill_kv_cache(dev, seq_lens, history_lens, dtype, idx):
    from dlcompiler_amd.kernels.fill_kv_cache import fill_kv_cache

    g = torch.Generator().manual_seed(0)
    H, D, bs = 8, 128, 64
    kv_lens = [s + h for s, h in zip(seq_lens, history_lens)]
    nblk = [_div_up(l, bs) for l in kv_lens]
    B = len(seq_lens)
    table = (torch.arange(B)[:, None] + torch.arange(max(nblk))[None, :] * B)
    ks = torch.rand((sum(seq_lens), H, D), generator=g).to(dtype)
    vs = torch.rand((sum(seq_lens), H, D), generator=g).to(dtype)
    kc = torch.zeros((B * max(nblk), bs, H, D), dtype=dtype)
    vc = torch.rand((B * max(nblk), bs, H, D), generator=g).to(dtype)
    q_len = torch.tensor(seq_lens)
    q_start = q_len.cumsum(0) - q_len
    rk, rv = od.fill_kv_cache(ks, vs, kc, vc, seq_lens, history_lens, table)
    kcd, vcd = kc.to(dev), vc.to(dev)
    # index tensors are read in the integer width they arrive in
    it = [torch.int64, torch.int32, torch.int16, torch.int32] if idx == "mixed" else [idx] * 4
    fill_kv_cache(ks.to(dev), vs.to(dev), kcd, vcd, q_start.to(it[0]).to(dev), q_len.to(it[1]).to(dev),
                  torch.tensor(kv_lens).to(it[2]).to(dev), max(seq_lens), table.to(it[3]).to(dev))
    assert torch.equal(kcd.cpu(), rk) and torch.equal(vcd.cpu(), rv)     # a copy: exact


def test_fill_kv_cache_odd_head_dims_and_views(dev):
    from dlcompiler_amd.kernels.fill_kv_cache import fill_kv_cache

    g = torch.Generator().manual_seed(1)
    seq_lens, hist, bs = [3, 20], [5, 0], 16
    kv = torch.rand((23, 3, 24 + 40), generator=g).half()       # K and V interleaved per head
    ks, vs = kv[..., :24], kv[..., 24:]                          # head dims 24 and 40, strided views
    kc, vc = torch.zeros((4, bs, 3, 24)).half(), torch.zeros((4, bs, 3, 40)).half()
    table = torch.tensor([[2, 0], [1, 3]])
    rk, rv = od.fill_kv_cache(ks, vs, kc, vc, seq_lens, hist, table)
    kvd = kv.to(dev)
    kcd, vcd = kc.to(dev), vc.to(dev)
    fill_kv_cache(kvd[..., :24], kvd[..., 24:], kcd, vcd, torch.tensor([0, 3]).to(dev),
                  torch.tensor(seq_lens).to(dev), torch.tensor([8, 20]).to(dev), 20, table.to(dev))
    assert torch.equal(kcd.cpu(), rk) and torch.equal(vcd.cpu(), rv)


# test_rms_norm.py:33-35: bf16, fp16 and fp32 on a (4, 8) input
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(4, 8), (3, 7, 4096), (64, 2048), (5, 11008), (2, 16384), (6, 12),
                                   (3, 1), (7, 77), (2, 16392), (2, 20000), (3, 4099)])
def test_rms_norm(dev, dtype, shape):
    from dlcompiler_amd.kernels.rms_norm import add_rms_norm, rms_norm

    g = torch.Generator().manual_seed(2)
    x = torch.rand(shape, generator=g).to(dtype)                 # reference fixture: torch.rand
    w = torch.rand(shape[-1], generator=g).to(dtype)
    ref = od.rms_norm(x, w, 1e-6)
    out = rms_norm(x.to(dev), w.to(dev), 1e-6).cpu()
    # the reference's tolerance is assert_close's default (fp16 1e-3, bf16 1.6e-2 relative);
    # the row sum is accumulated in a different order, which can flip the first of the two
    # roundings (normalise, then times weight) by one ulp -> allow two fp16 ulps
    tol = dict(rtol=2e-3, atol=1e-5) if dtype == torch.float16 else dict(rtol=1.6e-2, atol=1e-5)
    if dtype == torch.float32:  # assert_close's default for fp32 (1.3e-6) plus the sum order
        tol = dict(rtol=5e-6, atol=1e-6)
    torch.testing.assert_close(out, ref, **tol)
    res = torch.randn(shape, generator=g).to(dtype)
    rout, rres = od.rms_norm(x, w, 1e-6, residual=res)
    out2, res2 = rms_norm(x.to(dev), w.to(dev), 1e-6, residual=res.to(dev))
    assert torch.equal(res2.cpu(), rres)                          # one add, one rounding: exact
    torch.testing.assert_close(out2.cpu(), rout, **tol)
    x2d = x.reshape(-1, shape[-1])
    o3, r3 = add_rms_norm(x2d.to(dev), w.to(dev), 1e-6, res.reshape(-1, shape[-1]).to(dev))
    assert torch.equal(o3.cpu().reshape(shape), out2.cpu()) and torch.equal(r3.cpu().reshape(shape), res2.cpu())


# test_apply_rotary.py:71-90: heads (8,8)/(8,4), feature dim 16, bf16/fp16/fp32, random positions
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hq,hk,d", [(8, 8, 16), (8, 4, 16), (32, 8, 128), (5, 1, 64), (3, 2, 2),
                                     (4, 4, 6), (8, 2, 40), (2, 1, 100)])
def test_apply_rotary(dev, dtype, hq, hk, d):
    from dlcompiler_amd.kernels.apply_rotary_pos_emb import apply_rotary_pos_emb

    g = torch.Generator().manual_seed(3)
    T, max_pos = 45, 16
    q = torch.rand((T, hq, d), generator=g).to(dtype)
    k = torch.rand((T, hk, d), generator=g).to(dtype)
    pos = torch.randint(0, max_pos, (T,), generator=g)
    cos = torch.rand((max_pos, d), generator=g).to(dtype)[pos, None, :]
    sin = torch.rand((max_pos, d), generator=g).to(dtype)[pos, None, :]
    rq, rk = od.apply_rotary_pos_emb(q.float(), k.float(), cos.float(), sin.float())
    qe, ke = apply_rotary_pos_emb(q.to(dev), k.to(dev), cos.to(dev), sin.to(dev))
    tol = dict(rtol=1e-5, atol=1e-3) if dtype == torch.float16 else dict(rtol=1.6e-2, atol=1e-5)
    if dtype == torch.float32:  # products may be contracted into fused multiply-adds
        tol = dict(rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(qe.cpu().float(), rq, **tol)
    torch.testing.assert_close(ke.cpu().float(), rk, **tol)
    # and against the reference ground truth evaluated in the storage dtype
    gq, gk = od.apply_rotary_pos_emb(q, k, cos, sin)
    torch.testing.assert_close(qe.cpu(), gq, rtol=2e-2, atol=2e-2)
    # in place
    qd, kd = q.to(dev), k.to(dev)
    q2, k2 = apply_rotary_pos_emb(qd, kd, cos.to(dev), sin.to(dev), qd, kd)
    assert q2.data_ptr() == qd.data_ptr() and torch.equal(q2, qe) and torch.equal(k2, ke)
