"""Writes the golden fixtures in this directory:  python tests/golden/make_fixtures.py

The reference ships no data files and draws its test inputs from the device RNG, so there is
nothing to carry over; these fixtures are small seeded inputs (CPU generator) together with the
outputs of the CPU oracle, whose functions are pinned by tests/test_oracle_*.py.  They freeze
those outputs: a later change of the oracle, of a rounding point or of torch's CPU kernels shows
up as a fixture mismatch (tests/test_golden_fixtures.py, CPU half) instead of silently moving
the target of the GPU parity tests (GPU half of the same file).
"""
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import fixture_io as fio  # noqa: E402
from oracle import activation as oact  # noqa: E402
from oracle import attention as oatt  # noqa: E402
from oracle import decoder_ops as odec  # noqa: E402
from oracle import fp8 as ofp8  # noqa: E402
from oracle import fused_moe as ofm  # noqa: E402
from oracle import moe_gating as og  # noqa: E402

BF, HF = torch.bfloat16, torch.float16


def gen(seed):
    return torch.Generator().manual_seed(seed)


def silu():
    g = gen(100)
    xb = (torch.randn((7, 2 * 136), generator=g) * 3).to(BF)
    xb[0, :4] = torch.tensor([0.0, -0.0, 30.0, -30.0]).to(BF)
    xh = (torch.randn((5, 2 * 264), generator=g) * 3).to(HF)
    fio.save("silu_and_mul", x_bf16=xb, out_bf16=oact.silu_and_mul_fp32(xb),
             gt_bf16=oact.silu_and_mul(xb), x_f16=xh, out_f16=oact.silu_and_mul_fp32(xh))


def gating():
    g = gen(101)
    logits = torch.randn((50, 64), generator=g)
    logits[3] = 0.0                      # every expert ties: ids 0..5
    logits[4, 10] = logits[4, 20] = 5.0  # a tie at the top: 10 before 20
    w, ids = og.topk_softmax(logits, 6, True)
    w_raw, _ = og.topk_softmax(logits, 6, False)
    s, e, tot, cnt = og.align_block_size(ids, 16, 64)
    start, end = og.start_end(ids, 64)
    # the reference's fused gate kernel in its own output form (full softmax, one-hot masks)
    gates, masks = og.topk_gating_part1(logits, 6)
    assert torch.equal(masks.argmax(-1).t().to(torch.int32), ids)   # same selection as the index form
    fio.save("moe_gating", logits=logits, k=6, block=16, weights=w, weights_no_renorm=w_raw,
             ids=ids, sorted_token_ids=s, expert_ids=e, num_tokens_post_padded=tot, counts=cnt,
             exp_start=start, exp_end=end, gates=gates, masks=masks)


def prefill():
    g = gen(102)
    lens = [37, 130, 1, 64]
    T = sum(lens)
    q = torch.randn((T, 4, 64), generator=g).to(BF)
    k = torch.randn((T, 2, 64), generator=g).to(BF)
    v = torch.randn((T, 2, 64), generator=g).to(BF)
    seq = torch.tensor(lens, dtype=torch.int32)
    start = (seq.cumsum(0) - seq).to(torch.int32)
    fio.save("prefill_attention", q=q, k=k, v=v, b_start_loc=start, b_seq_len=seq,
             out=oatt.prefill_attention(q, k, v, start, seq))


def paged():
    g = gen(103)
    page, hq, hkv, d = 16, 8, 2, 128
    ctx = [1, 70, 200, 16]
    ks = [torch.randn((l, hkv, d), generator=g).to(BF) for l in ctx]
    vs = [torch.randn((l, hkv, d), generator=g).to(BF) for l in ctx]
    kc, vc, table = oatt.make_paged_cache(ks, vs, page, seed=7, dtype=BF)
    # (cache rows no context owns hold NaN: a read past a context shows in the output)
    kv_len = torch.tensor(ctx, dtype=torch.int32)
    qd = torch.randn((len(ctx), hq, d), generator=g).to(BF)
    fio.save("paged_decode", q=qd, k_cache=kc, v_cache=vc, block_table=table, kv_len=kv_len,
             out=oatt.paged_decode(qd, kc, vc, table, kv_len),
             window=24, softcap=30.0,
             out_window_softcap=oatt.paged_decode(qd, kc, vc, table, kv_len, window=24,
                                                  softcap=30.0))
    # prefill with history over the same caches: the last q_len positions of each context
    q_len = torch.tensor([1, 40, 33, 16], dtype=torch.int32)
    q_start = (q_len.cumsum(0) - q_len).to(torch.int32)
    qp = torch.randn((int(q_len.sum()), hq, d), generator=g).to(BF)
    fio.save("paged_prefill", q=qp, k_cache=kc, v_cache=vc, block_table=table, kv_len=kv_len,
             q_start_loc=q_start, q_len=q_len,
             out=oatt.paged_prefill(qp, kc, vc, table, q_start, q_len, kv_len),
             window=24,
             out_window=oatt.paged_prefill(qp, kc, vc, table, q_start, q_len, kv_len, window=24))


def decoder_ops():
    g = gen(104)
    seq_lens, hist = (3, 1, 20), (0, 15, 30)
    H, D, bs = 2, 64, 16
    kv = [s + h for s, h in zip(seq_lens, hist)]
    nblk = max(-(-l // bs) for l in kv)
    B = len(seq_lens)
    table = (torch.arange(B)[:, None] + torch.arange(nblk)[None, :] * B).to(torch.int32)
    ks = torch.randn((sum(seq_lens), H, D), generator=g).to(BF)
    vs = torch.randn((sum(seq_lens), H, D), generator=g).to(BF)
    kc = torch.randn((B * nblk, bs, H, D), generator=g).to(BF)
    vc = torch.randn((B * nblk, bs, H, D), generator=g).to(BF)
    rk, rv = odec.fill_kv_cache(ks, vs, kc, vc, seq_lens, hist, table)
    ql = torch.tensor(seq_lens, dtype=torch.int32)
    fio.save("fill_kv_cache", k_states=ks, v_states=vs, k_cache=kc, v_cache=vc,
             q_start_loc=(ql.cumsum(0) - ql).to(torch.int32), q_len=ql,
             kv_len=torch.tensor(kv, dtype=torch.int32), block_table=table, k_cache_out=rk,
             v_cache_out=rv)

    x = torch.randn((5, 256), generator=g).to(BF)
    w = torch.rand((256,), generator=g).to(BF)
    res = torch.randn((5, 256), generator=g).to(BF)
    out_add, res_out = odec.rms_norm(x, w, 1e-6, residual=res)
    # a row length that is no whole number of 16-byte vectors (the element-wise kernel)
    x77 = torch.randn((3, 77), generator=g).to(HF)
    w77 = torch.rand((77,), generator=g).to(HF)
    r77 = torch.randn((3, 77), generator=g).to(HF)
    o77, ro77 = odec.rms_norm(x77, w77, 1e-6, residual=r77)
    fio.save("rms_norm", x=x, weight=w, residual=res, eps=1e-6, out=odec.rms_norm(x, w, 1e-6),
             out_add=out_add, residual_out=res_out, x77=x77, weight77=w77, residual77=r77,
             out77=odec.rms_norm(x77, w77, 1e-6), out_add77=o77, residual_out77=ro77)

    T, hq, hk, d = 6, 4, 2, 64
    q = torch.randn((T, hq, d), generator=g).to(HF)
    k = torch.randn((T, hk, d), generator=g).to(HF)
    ang = torch.rand((T, 1, d // 2), generator=g) * 6.28
    cos = torch.cat((ang.cos(), ang.cos()), -1).to(HF)
    sin = torch.cat((ang.sin(), ang.sin()), -1).to(HF)
    rq, rk_ = odec.apply_rotary_pos_emb(q.float(), k.float(), cos.float(), sin.float())
    # head size 6: not a multiple of a 16-byte vector (the element-wise kernel)
    q6 = torch.randn((T, 3, 6), generator=g).to(BF)
    k6 = torch.randn((T, 1, 6), generator=g).to(BF)
    a6 = torch.rand((T, 1, 3), generator=g) * 6.28
    c6 = torch.cat((a6.cos(), a6.cos()), -1).to(BF)
    s6 = torch.cat((a6.sin(), a6.sin()), -1).to(BF)
    rq6, rk6 = odec.apply_rotary_pos_emb(q6.float(), k6.float(), c6.float(), s6.float())
    fio.save("apply_rotary_pos_emb", q=q, k=k, cos=cos, sin=sin, q_embed_f32=rq, k_embed_f32=rk_,
             q6=q6, k6=k6, cos6=c6, sin6=s6, q6_embed_f32=rq6, k6_embed_f32=rk6)


def moe():
    g = gen(105)
    T, H, I, E, k = 9, 128, 128, 4, 2
    x = torch.randn((T, H), generator=g).to(BF)
    logits = torch.randn((T, E), generator=g)
    w1 = (torch.randn((E, 2 * I, H), generator=g) * 0.05)
    w2 = (torch.randn((E, H, I), generator=g) * 0.05)
    tw, ids = og.topk_softmax(logits, k, True)
    fio.save("fused_moe_bf16", hidden=x, w1=w1.to(BF), w2=w2.to(BF), topk_weights=tw,
             topk_ids=ids, topk=k, out=ofm.fused_moe(x, w1.to(BF), w2.to(BF), tw, ids))
    xq, xs = ofp8.per_token_group_quant(x)
    w1q, w1s = ofp8.block_quant_weight(w1)
    w2q, w2s = ofp8.block_quant_weight(w2)
    fio.save("fused_moe_fp8", hidden=x, hidden_q=xq, hidden_scale=xs, w1_q=w1q, w1_s=w1s,
             w2_q=w2q, w2_s=w2s, topk_weights=tw, topk_ids=ids, topk=k,
             out=ofm.fused_moe_fp8(x, w1q, w1s, w2q, w2s, tw, ids))


def launcher():
    # the reference's grouped-GEMM launcher case in small (test_fused_moe.py:17-145)
    g = gen(106)
    M, K, N, E, k = 24, 64, 16, 3, 2
    A = ((torch.rand((M, K), generator=g) - 0.5) / 2).to(HF)
    B = ((torch.rand((E, N, K), generator=g) - 0.5) / 2).to(HF)
    weights, idx = torch.rand((M, E), generator=g).to(HF).topk(k, dim=-1)
    sorted_idx = idx.flatten().argsort(stable=True)
    start, end = og.start_end(idx, E)
    fio.save("moe_launcher", a=A, b=B, weights=weights, topk_idx=idx, sorted_idx=sorted_idx,
             exp_start=start, exp_end=end, top_k=k, out=ofm.grouped_gemm_launcher(A, B, idx, weights))


if __name__ == "__main__":
    torch.set_num_threads(1)
    for make in (silu, gating, prefill, paged, decoder_ops, moe, launcher):
        make()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
