"""Pins oracle.decoder_ops on the CPU: library routines and closed forms."""
import torch
import torch.nn.functional as F

from oracle import decoder_ops as od


def test_rms_norm_matches_library_and_closed_form():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((5, 64), generator=g)
    w = torch.rand(64, generator=g)
    torch.testing.assert_close(od.rms_norm(x, w, 1e-6), F.rms_norm(x, (64,), w, 1e-6), rtol=1e-5, atol=1e-6)
    const = torch.full((2, 8), 3.0)
    assert torch.allclose(od.rms_norm(const, torch.ones(8), 0.0), torch.ones(2, 8))   # x / |x|
    out, new_res = od.rms_norm(x, w, 1e-6, residual=x)
    assert torch.equal(new_res, 2 * x)
    torch.testing.assert_close(out, od.rms_norm(x, w, 1e-6 / 4), rtol=1e-5, atol=1e-6)  # scale invariance


def test_rotary_is_a_rotation():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn((7, 3, 16), generator=g), torch.randn((7, 2, 16), generator=g)
    theta = torch.rand((7, 1, 8), generator=g) * 6.28
    cos, sin = torch.cos(theta).repeat(1, 1, 2), torch.sin(theta).repeat(1, 1, 2)
    qe, ke = od.apply_rotary_pos_emb(q, k, cos, sin)
    # pairs (d, d + 8) rotate by theta_d: norms are preserved and the complex form agrees
    torch.testing.assert_close(qe.norm(dim=-1), q.norm(dim=-1))
    zc = torch.complex(q[..., :8], q[..., 8:]) * torch.polar(torch.ones_like(theta), theta)
    torch.testing.assert_close(qe[..., :8], zc.real)
    torch.testing.assert_close(qe[..., 8:], zc.imag)
    back, _ = od.apply_rotary_pos_emb(qe, ke, cos, -sin)
    torch.testing.assert_close(back, q, rtol=1e-5, atol=1e-5)


def test_fill_kv_cache_matches_reference_loop_structure():
    # the reference ground truth copies page-sized slices (test_fill_kv_cache.py:109-137);
    # restated here slice-wise and compared with the per-token oracle
    g = torch.Generator().manual_seed(2)
    seq_lens, hist = [1, 8, 16, 24], [1, 16, 31, 24]
    bs, H, D = 16, 2, 8
    blocks = [-(-(s + h) // bs) for s, h in zip(seq_lens, hist)]
    table = torch.arange(4)[:, None] + torch.arange(max(blocks))[None, :] * 4
    ks, vs = torch.randn((sum(seq_lens), H, D), generator=g), torch.randn((sum(seq_lens), H, D), generator=g)
    kc, vc = torch.zeros((4 * max(blocks), bs, H, D)), torch.randn((4 * max(blocks), bs, H, D), generator=g)
    ok, ov = od.fill_kv_cache(ks, vs, kc, vc, seq_lens, hist, table)
    rk, rv = kc.clone(), vc.clone()
    at = 0
    for b, (s, h) in enumerate(zip(seq_lens, hist)):
        k_state, v_state = ks[at:at + s], vs[at:at + s]
        at += s
        block_id, start = (h + 1 + bs - 1) // bs - 1, h % bs
        while k_state.shape[0] > 0:
            n = min(bs - start, k_state.shape[0])
            rk[table[b, block_id], start:start + n] = k_state[:n]
            rv[table[b, block_id], start:start + n] = v_state[:n]
            k_state, v_state, block_id, start = k_state[n:], v_state[n:], block_id + 1, 0
    assert torch.equal(ok, rk) and torch.equal(ov, rv)
