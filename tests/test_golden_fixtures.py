"""The committed fixtures under tests/golden/ (small seeded inputs + CPU-oracle outputs).

CPU half: the oracle still reproduces every stored output (integers and bytes bit for bit,
floats to one unit of the storage type), so the target of the GPU parity tests cannot drift
unnoticed.  GPU half: the HIP path, through the C ABI, against the stored outputs to the same
tolerances as the parity tests (integers bit-exact, gating weights 1e-6, 16-bit outputs 2e-2,
fp8 MoE 3e-2 relative).
"""
import importlib.util
import os

import pytest
import torch

from oracle import activation as oact
from oracle import attention as oatt
from oracle import decoder_ops as odec
from oracle import fp8 as ofp8
from oracle import fused_moe as ofm
from oracle import moe_gating as og

_spec = importlib.util.spec_from_file_location(
    "fixture_io", os.path.join(os.path.dirname(__file__), "golden", "fixture_io.py"))
fio = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(fio)

NAMES = ["silu_and_mul", "moe_gating", "prefill_attention", "paged_decode", "paged_prefill",
         "fill_kv_cache", "rms_norm", "apply_rotary_pos_emb", "fused_moe_bf16", "fused_moe_fp8",
         "moe_launcher"]


def _ulp(dtype):
    return {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}.get(dtype, 1e-5)


def _same(got, want):
    assert got.dtype == want.dtype and got.shape == want.shape
    if want.dtype.is_floating_point and want.dtype != torch.float8_e4m3fn:
        u = _ulp(want.dtype)
        torch.testing.assert_close(got.float(), want.float(), rtol=2 * u, atol=2 * u,
                                   equal_nan=True)
    else:
        assert torch.equal(got.view(torch.uint8) if want.dtype == torch.float8_e4m3fn else got,
                           want.view(torch.uint8) if want.dtype == torch.float8_e4m3fn else want)


def test_every_fixture_is_present():
    for n in NAMES:
        assert os.path.exists(fio.path(n)), "run python tests/golden/make_fixtures.py"
        assert os.path.getsize(fio.path(n)) < (1 << 20)


# ------------------------------------------------------------------ CPU: oracle vs fixtures
def test_oracle_reproduces_silu():
    f = fio.load("silu_and_mul")
    _same(oact.silu_and_mul_fp32(f["x_bf16"]), f["out_bf16"])
    _same(oact.silu_and_mul(f["x_bf16"]), f["gt_bf16"])
    _same(oact.silu_and_mul_fp32(f["x_f16"]), f["out_f16"])


def test_oracle_reproduces_gating():
    f = fio.load("moe_gating")
    w, ids = og.topk_softmax(f["logits"], f["k"], True)
    assert torch.equal(ids, f["ids"])
    assert ids[3].tolist() == [0, 1, 2, 3, 4, 5] and ids[4, :2].tolist() == [10, 20]   # the ties
    torch.testing.assert_close(w, f["weights"], rtol=1e-6, atol=0)
    torch.testing.assert_close(og.topk_softmax(f["logits"], f["k"], False)[0],
                               f["weights_no_renorm"], rtol=1e-6, atol=0)
    s, e, tot, cnt = og.align_block_size(f["ids"], f["block"], 64)
    assert torch.equal(s, f["sorted_token_ids"]) and torch.equal(e, f["expert_ids"])
    assert torch.equal(tot, f["num_tokens_post_padded"]) and torch.equal(cnt, f["counts"])
    start, end = og.start_end(f["ids"], 64)
    assert torch.equal(start, f["exp_start"]) and torch.equal(end, f["exp_end"])
    gates, masks = og.topk_gating_part1(f["logits"], f["k"])
    torch.testing.assert_close(gates, f["gates"], rtol=1e-6, atol=0)
    assert torch.equal(masks, f["masks"])


def test_oracle_reproduces_attention():
    f = fio.load("prefill_attention")
    _same(oatt.prefill_attention(f["q"], f["k"], f["v"], f["b_start_loc"], f["b_seq_len"]), f["out"])
    f = fio.load("paged_decode")
    args = (f["q"], f["k_cache"], f["v_cache"], f["block_table"], f["kv_len"])
    _same(oatt.paged_decode(*args), f["out"])
    _same(oatt.paged_decode(*args, window=f["window"], softcap=f["softcap"]), f["out_window_softcap"])
    f = fio.load("paged_prefill")
    args = (f["q"], f["k_cache"], f["v_cache"], f["block_table"], f["q_start_loc"], f["q_len"],
            f["kv_len"])
    _same(oatt.paged_prefill(*args), f["out"])
    _same(oatt.paged_prefill(*args, window=f["window"]), f["out_window"])


def test_oracle_reproduces_decoder_ops():
    f = fio.load("fill_kv_cache")
    seq = f["q_len"].tolist()
    hist = (f["kv_len"] - f["q_len"]).tolist()
    rk, rv = odec.fill_kv_cache(f["k_states"], f["v_states"], f["k_cache"], f["v_cache"], seq, hist,
                                f["block_table"])
    assert torch.equal(rk, f["k_cache_out"]) and torch.equal(rv, f["v_cache_out"])
    f = fio.load("rms_norm")
    _same(odec.rms_norm(f["x"], f["weight"], f["eps"]), f["out"])
    out, res = odec.rms_norm(f["x"], f["weight"], f["eps"], residual=f["residual"])
    _same(out, f["out_add"])
    assert torch.equal(res, f["residual_out"])
    _same(odec.rms_norm(f["x77"], f["weight77"], f["eps"]), f["out77"])
    out, res = odec.rms_norm(f["x77"], f["weight77"], f["eps"], residual=f["residual77"])
    _same(out, f["out_add77"])
    assert torch.equal(res, f["residual_out77"])
    f = fio.load("apply_rotary_pos_emb")
    rq, rk = odec.apply_rotary_pos_emb(f["q"].float(), f["k"].float(), f["cos"].float(),
                                       f["sin"].float())
    _same(rq, f["q_embed_f32"])
    _same(rk, f["k_embed_f32"])
    rq, rk = odec.apply_rotary_pos_emb(f["q6"].float(), f["k6"].float(), f["cos6"].float(),
                                       f["sin6"].float())
    _same(rq, f["q6_embed_f32"])
    _same(rk, f["k6_embed_f32"])


def test_oracle_reproduces_moe():
    f = fio.load("fused_moe_bf16")
    _same(ofm.fused_moe(f["hidden"], f["w1"], f["w2"], f["topk_weights"], f["topk_ids"]), f["out"])
    f = fio.load("fused_moe_fp8")
    q, s = ofp8.per_token_group_quant(f["hidden"])
    _same(q, f["hidden_q"])
    assert torch.equal(s, f["hidden_scale"])
    _same(ofm.fused_moe_fp8(f["hidden"], f["w1_q"], f["w1_s"], f["w2_q"], f["w2_s"],
                            f["topk_weights"], f["topk_ids"]), f["out"])
    f = fio.load("moe_launcher")
    _same(ofm.grouped_gemm_launcher(f["a"], f["b"], f["topk_idx"], f["weights"]), f["out"])
    start, end = og.start_end(f["topk_idx"], f["b"].shape[0])
    assert torch.equal(start, f["exp_start"]) and torch.equal(end, f["exp_end"])


# ------------------------------------------------------------------ GPU: HIP path vs fixtures
def _close16(got, want, tol=2e-2):
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=tol, atol=tol)


@pytest.mark.gpu
def test_hip_silu_matches_fixture(dev):
    from dlcompiler_amd.kernels.activation import silu_and_mul

    f = fio.load("silu_and_mul")
    assert torch.equal(silu_and_mul(f["x_bf16"].to(dev)).cpu(), f["out_bf16"])   # same rounding points
    _close16(silu_and_mul(f["x_bf16"].to(dev)), f["gt_bf16"])
    torch.testing.assert_close(silu_and_mul(f["x_f16"].to(dev)).cpu(), f["out_f16"], rtol=1e-3,
                               atol=1e-3)


@pytest.mark.gpu
def test_hip_gating_matches_fixture(dev):
    from dlcompiler_amd.kernels.fused_moe import get_start_end
    from dlcompiler_amd.kernels.moe_gating import (moe_align_block_size, moe_topk_softmax,
                                                   moe_topk_softmax_align)

    f = fio.load("moe_gating")
    logits = f["logits"].to(dev)
    w, ids = moe_topk_softmax(logits, f["k"], True)
    assert ids.dtype == torch.int32 and torch.equal(ids.cpu(), f["ids"])
    torch.testing.assert_close(w.cpu(), f["weights"], rtol=1e-6, atol=0)
    torch.testing.assert_close(moe_topk_softmax(logits, f["k"], False)[0].cpu(),
                               f["weights_no_renorm"], rtol=1e-6, atol=0)
    s, e, tot, cnt = moe_align_block_size(ids, f["block"], 64, return_counts=True)
    fused = moe_topk_softmax_align(logits, f["k"], f["block"])
    for got in ((s, e, tot), fused[2:]):
        assert torch.equal(got[0].cpu(), f["sorted_token_ids"])
        assert torch.equal(got[1].cpu(), f["expert_ids"])
        assert torch.equal(got[2].cpu().reshape(-1), f["num_tokens_post_padded"])
    assert torch.equal(cnt.cpu(), f["counts"]) and torch.equal(fused[1].cpu(), f["ids"])
    start, end = get_start_end(ids, torch.empty(0, dtype=torch.int64, device=dev), 64)
    assert torch.equal(start.cpu(), f["exp_start"]) and torch.equal(end.cpu(), f["exp_end"])
    from dlcompiler_amd.kernels.topk_gating_fwd_part1 import call as gating_part1

    gates, masks = gating_part1(logits, f["k"])
    torch.testing.assert_close(gates.cpu(), f["gates"], rtol=2e-6, atol=0)
    assert torch.equal(masks.cpu(), f["masks"])


@pytest.mark.gpu
def test_hip_attention_matches_fixtures(dev):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    f = fio.load("prefill_attention")
    o = torch.zeros_like(f["q"], device=dev)
    context_attention_fwd(f["q"].to(dev), f["k"].to(dev), f["v"].to(dev), o, f["b_start_loc"].to(dev),
                          f["b_seq_len"].to(dev), int(f["b_seq_len"].max()))
    _close16(o, f["out"])

    f = fio.load("paged_decode")
    B = f["q"].shape[0]
    ones = torch.ones(B, dtype=torch.int32, device=dev)
    start = torch.arange(B, dtype=torch.int32, device=dev)
    for key, kw in (("out", {}), ("out_window_softcap", dict(window_size=f["window"],
                                                           logit_softcapping=f["softcap"]))):
        o = torch.zeros_like(f["q"], device=dev)
        paged_attention_fwd(f["q"].to(dev), f["k_cache"].to(dev), f["v_cache"].to(dev), o,
                            f["block_table"].to(dev), start, ones, f["kv_len"].to(dev), 1, **kw)
        _close16(o, f[key])

    f = fio.load("paged_prefill")
    for key, kw in (("out", {}), ("out_window", dict(window_size=f["window"]))):
        o = torch.zeros_like(f["q"], device=dev)
        paged_attention_fwd(f["q"].to(dev), f["k_cache"].to(dev), f["v_cache"].to(dev), o,
                            f["block_table"].to(dev), f["q_start_loc"].to(dev), f["q_len"].to(dev),
                            f["kv_len"].to(dev), int(f["q_len"].max()), **kw)
        _close16(o, f[key])


@pytest.mark.gpu
def test_hip_decoder_ops_match_fixtures(dev):
    from dlcompiler_amd.kernels.apply_rotary_pos_emb import apply_rotary_pos_emb
    from dlcompiler_amd.kernels.fill_kv_cache import fill_kv_cache
    from dlcompiler_amd.kernels.rms_norm import rms_norm

    f = fio.load("fill_kv_cache")
    kc, vc = f["k_cache"].to(dev), f["v_cache"].to(dev)
    fill_kv_cache(f["k_states"].to(dev), f["v_states"].to(dev), kc, vc, f["q_start_loc"].to(dev),
                  f["q_len"].to(dev), f["kv_len"].to(dev), int(f["q_len"].max()),
                  f["block_table"].to(dev))
    assert torch.equal(kc.cpu(), f["k_cache_out"]) and torch.equal(vc.cpu(), f["v_cache_out"])

    f = fio.load("rms_norm")
    tol = dict(rtol=1.6e-2, atol=1e-5)
    torch.testing.assert_close(rms_norm(f["x"].to(dev), f["weight"].to(dev), f["eps"]).cpu(),
                               f["out"], **tol)
    out, res = rms_norm(f["x"].to(dev), f["weight"].to(dev), f["eps"], residual=f["residual"].to(dev))
    assert torch.equal(res.cpu(), f["residual_out"])
    torch.testing.assert_close(out.cpu(), f["out_add"], **tol)
    tol77 = dict(rtol=2e-3, atol=1e-5)                      # fp16 rows of 77 elements
    torch.testing.assert_close(rms_norm(f["x77"].to(dev), f["weight77"].to(dev), f["eps"]).cpu(),
                               f["out77"], **tol77)
    out, res = rms_norm(f["x77"].to(dev), f["weight77"].to(dev), f["eps"], residual=f["residual77"].to(dev))
    assert torch.equal(res.cpu(), f["residual_out77"])
    torch.testing.assert_close(out.cpu(), f["out_add77"], **tol77)

    f = fio.load("apply_rotary_pos_emb")
    qe, ke = apply_rotary_pos_emb(f["q"].to(dev), f["k"].to(dev), f["cos"].to(dev), f["sin"].to(dev))
    torch.testing.assert_close(qe.cpu().float(), f["q_embed_f32"], rtol=1e-5, atol=2e-3)
    torch.testing.assert_close(ke.cpu().float(), f["k_embed_f32"], rtol=1e-5, atol=2e-3)
    qe, ke = apply_rotary_pos_emb(f["q6"].to(dev), f["k6"].to(dev), f["cos6"].to(dev), f["sin6"].to(dev))
    torch.testing.assert_close(qe.cpu().float(), f["q6_embed_f32"], rtol=1.6e-2, atol=1e-2)
    torch.testing.assert_close(ke.cpu().float(), f["k6_embed_f32"], rtol=1.6e-2, atol=1e-2)


@pytest.mark.gpu
def test_hip_moe_matches_fixtures(dev):
    from dlcompiler_amd.kernels.fused_moe import fused_moe, fused_moe_fp8, per_token_group_quant_fp8

    f = fio.load("fused_moe_bf16")
    out = fused_moe(f["hidden"].to(dev), f["w1"].to(dev), f["w2"].to(dev), f["topk_weights"].to(dev),
                    f["topk_ids"].to(dev), f["topk"])
    _close16(out, f["out"])

    f = fio.load("fused_moe_fp8")
    q, s = per_token_group_quant_fp8(f["hidden"].to(dev))
    assert torch.equal(q.cpu().view(torch.uint8), f["hidden_q"].view(torch.uint8))
    assert torch.equal(s.cpu(), f["hidden_scale"])
    out = fused_moe_fp8(f["hidden"].to(dev), f["w1_q"].to(dev), f["w1_s"].to(dev), f["w2_q"].to(dev),
                        f["w2_s"].to(dev), f["topk_weights"].to(dev), f["topk_ids"].to(dev), f["topk"])
    ref = f["out"].double()
    assert ((out.cpu().double() - ref).norm() / ref.norm()).item() <= 3e-2

    from dlcompiler_amd.kernels.fused_moe import fused_moe_kernel_launcher

    f = fio.load("moe_launcher")
    C = torch.zeros(f["out"].shape, dtype=f["out"].dtype, device=dev)
    fused_moe_kernel_launcher(f["a"].to(dev), f["b"].to(dev), C, f["sorted_idx"].to(dev),
                              f["exp_start"].to(dev), f["exp_end"].to(dev), f["weights"].to(dev),
                              enable_weights=True, top_k=f["top_k"], num_tokens=f["a"].shape[0])
    torch.testing.assert_close(C.cpu(), f["out"])
