#!/usr/bin/env python3
"""Benchmark of the dlBLAS inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Runs the five benchmark configurations (fused silu_and_mul, MoE gating + alignment,
varlen causal prefill attention, paged decode attention, fp8 fused-MoE MLP), the reference's own
bf16 fused_moe at the config-5 shape and four neighbouring decoder-layer operators (add + RMSNorm,
rotary embedding, KV-cache fill, paged prefill) on synthetic,
seeded inputs that are resident in HBM before the timed region, and prints ONE JSON line.
A "step" is one call of an operator's public entry point on one batch.  The top-level
`metric`/`value`/`roofline`/`cpu_baseline` describe the primary workload (--workload, default
the fp8 fused MoE); `workloads` carries the same figures for every configuration.

For each workload:
  value      algorithmic work / wall time of the K = --steps back-to-back steps, bracketed by one
             event pair on the launch stream, after max(--warmup, 10) untimed steps
  timing     100 further iterations in 20 batches: median / p10 / p90 of the per-step time
  roofline   the dominant kernel: algorithmic bytes (or FLOPs) per launch / its median launch
             duration from events on the launch stream (for the single-kernel workloads a step
             IS that launch; the MoE GEMMs and the two gating kernels are timed in passes of
             their own); `traffic` (HBM bytes per launch from rocprofv3 --pmc, a separate run)
             is read from profiles/hbm_traffic.json when a measurement has been committed
  cpu_baseline  the CPU oracle (a port of the reference's PyTorch ground truth) timed on a
             bounded sample of the same workload on this host's cores (model string included)
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_FP8_TFLOPS = 5000.0


def _gen(seed):
    return torch.Generator().manual_seed(seed)


class Timer:
    """Events on the current (launch) stream."""

    def __init__(self):
        self.pairs = []

    def start(self):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        return ev

    def stop(self, ev0):
        ev1 = torch.cuda.Event(enable_timing=True)
        ev1.record()
        self.pairs.append((ev0, ev1))

    def mean_ms(self):
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in self.pairs) / max(len(self.pairs), 1)


MIN_WARMUP = 10       # warm-up iterations before any timed region, whatever --warmup says
MIN_WARMUP_S = 0.05   # ... and at least this much wall time of warm-up steps
STAT_ITERS = 100      # iterations behind the median / p10 / p90 figures
STAT_BATCHES = 20


def _percentile(sorted_vals, q):
    if not sorted_vals:
        return None
    pos = q * (len(sorted_vals) - 1)
    lo, hi = int(math.floor(pos)), int(math.ceil(pos))
    return sorted_vals[lo] + (sorted_vals[hi] - sorted_vals[lo]) * (pos - lo)


def _time_steps(step, steps, warmup):
    """step(i) launches one step.  Returns (ms_per_step, stats).

    ms_per_step: the K = `steps` timed steps are bracketed by one event before and one after on
    the launch stream, and nothing else is recorded inside the region (an event pair around every
    step costs about 10 us of host time and 7 us of GPU time per step -- a quarter of the shortest
    workload).  At least MIN_WARMUP untimed steps and MIN_WARMUP_S seconds of them run first.
    stats: STAT_ITERS further iterations in STAT_BATCHES batches, one event pair per batch; the
    median / p10 / p90 are over the per-step times of the batches (batch time / batch size).  For
    a single-kernel workload a step is that kernel's launch, launch gaps included."""
    t0 = time.perf_counter()
    n_warm = warmup if COUNTER_PASS else max(warmup, MIN_WARMUP)
    for i in range(n_warm):
        step(i)
    torch.cuda.synchronize()
    # a workload of a few microseconds per step has not brought the chip out of its idle clocks
    # after ten steps: keep warming (untimed) until MIN_WARMUP_S of wall time have passed
    while not COUNTER_PASS and time.perf_counter() - t0 < MIN_WARMUP_S and n_warm < 20000:
        for i in range(10):
            step(n_warm + i)
        n_warm += 10
        torch.cuda.synchronize()
    t_all = Timer()
    ev = t_all.start()
    for i in range(steps):
        step(i)
    t_all.stop(ev)
    torch.cuda.synchronize()
    ms = t_all.mean_ms() / steps
    return ms, _batch_stats(step)


COUNTER_PASS = False  # --counters: a run under a hardware-counter pass keeps launches few


def _batch_stats(step, iters=None, batches=None):
    iters = iters or (4 if COUNTER_PASS else STAT_ITERS)
    batches = batches or (2 if COUNTER_PASS else STAT_BATCHES)
    per = max(1, -(-iters // batches))
    tb = Timer()
    n = 0
    for _ in range(batches):
        ev = tb.start()
        for _ in range(per):
            step(n)
            n += 1
        tb.stop(ev)
    torch.cuda.synchronize()
    vals = sorted(a.elapsed_time(b) / per for a, b in tb.pairs)
    return {"iterations": n, "batch": per, "median_ms": _percentile(vals, 0.5),
            "p10_ms": _percentile(vals, 0.1), "p90_ms": _percentile(vals, 0.9)}


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _cpu_info(cores=None):
    return {"cores": cores if cores is not None else torch.get_num_threads(),
            "cpu_model": _cpu_model(), "cpu_count": os.cpu_count()}


def _cpu_time(fn, reps=3, warm=None):
    """Seconds per call of a CPU-oracle leg: one untimed warm-up call (``warm`` if given, a cheaper
    call that touches the same code paths, else ``fn`` itself), then the median of ``reps`` timed
    calls."""
    (warm or fn)()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


TRAFFIC_NOTE = ("traffic = bytes that missed the L2 per launch (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, "
                "scaled by a copy kernel of known size), read from profiles/hbm_traffic.json -- a separate, "
                "committed run, not this one; hits in the 256 MB Infinity Cache are inside it, so it is an "
                "upper bound of the HBM bytes")


def _traffic(name):
    """HBM bytes per launch of the named kernel from the committed rocprofv3 --pmc summary (a
    separate run: counters cannot be read inside this process), or None."""
    if name is None:
        return None
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(name)
    except (OSError, ValueError):
        return None


# --------------------------------------------------------------------------------------
# workloads
# --------------------------------------------------------------------------------------
def wl_silu(dev, steps, warmup, cpu):
    from dlcompiler_amd.kernels.activation import silu_and_mul

    M, N = 8192, 11008
    nbuf = 3  # rotate > 2 x 256 MB of distinct buffers so nothing is served from cache
    x0 = torch.randn((M, 2 * N), generator=_gen(0)).bfloat16()
    xs = [x0.to(dev)] + [x0.to(dev).roll(i, 0) for i in range(1, nbuf)]
    outs = [torch.empty((M, N), dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
    bytes_ = M * 2 * N * 2 + M * N * 2

    ms, st = _time_steps(lambda i: silu_and_mul(xs[i % nbuf], outs[i % nbuf]), steps, warmup)
    ms_kernel = st["median_ms"]
    res = {
        "metric": "silu_and_mul HBM GB/s", "unit": "GB/s", "value": bytes_ / ms / 1e6,
        "ms_per_step": ms, "timing": st, "dtype": "bf16",
        "config": {"workload": "silu_and_mul bf16 [8192, 2x11008] N(0,1) seed 0"},
        "roofline": {"kernel": "silu_and_mul_vec16", "bound": "hbm",
                     "achieved": bytes_ / ms_kernel / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": bytes_ / ms_kernel / 1e6 / PEAK_HBM_GBS,
                     "traffic": _traffic("silu_and_mul")},
    }
    if cpu:
        from oracle import activation as oa

        rows = 1024
        sample = x0[:rows]
        dt = _cpu_time(lambda: oa.silu_and_mul(sample), warm=lambda: oa.silu_and_mul(sample[:64]))
        res["cpu_baseline"] = {"value": bytes_ * rows / M / dt / 1e9, "unit": "GB/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"{rows} of {M} rows, 1 warm-up + median of 3 reps"}
    return res


def _graph_replay_ms(fn, steps, warmup, label):
    if COUNTER_PASS:
        return None
    """Mean time of one replay of ``fn`` captured into a HIP graph (optional extra figure: the
    public calls with no Python or launch latency between their kernels).  None if capture fails."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            out = fn()
        for _ in range(warmup):
            g.replay()
        torch.cuda.synchronize()
        t = Timer()
        ev = t.start()
        for _ in range(steps):
            g.replay()
        t.stop(ev)
        ms = t.mean_ms() / steps
        del out, g
        return ms
    except Exception as exc:  # graph capture is optional reporting
        print(f"[bench] {label} graph replay skipped: {exc}", file=sys.stderr)
        return None


def wl_gating(dev, steps, warmup, cpu):
    from dlcompiler_amd.kernels.moe_gating import (moe_align_block_size, moe_topk_softmax,
                                                   moe_topk_softmax_align)

    T, E, K, BLK = 16384, 64, 6, 64
    logits_cpu = torch.randn((T, E), generator=_gen(1))
    logits = logits_cpu.to(dev)

    def step(i):  # router + alignment as one native call (two launches)
        return moe_topk_softmax_align(logits, K, BLK)

    def step_two_calls(i):  # the same result from the two separate operators (three launches)
        w, ids = moe_topk_softmax(logits, K)
        return moe_align_block_size(ids, BLK, E)

    npad = step(0)[4]
    l_pad = int(npad.item())
    bytes_ = (T * E * 4 + T * K * 4 * 2 + T * K * 4 + 4 * l_pad + 4 * l_pad // BLK + E * 4 + 4)
    ms, st = _time_steps(step, steps, warmup)
    ms_two, _ = _time_steps(step_two_calls, steps, warmup)

    # GPU time of the call itself (its two kernels and the gap between them), without the host
    # between calls: N calls captured into one HIP graph, replayed; a graph of ONE call replayed
    # shows what a graph launch itself costs on this stack
    calls = 20
    graph_ms = _graph_replay_ms(lambda: [step(0) for _ in range(calls)][-1], 20, 5, "gating")
    graph1_ms = _graph_replay_ms(lambda: step(0), 20, 5, "gating (one call per graph)")
    ms_gpu = graph_ms / calls if graph_ms is not None else st["median_ms"]
    res = {
        "metric": "MoE gating HBM GB/s", "unit": "GB/s", "value": bytes_ / ms / 1e6,
        "ms_per_step": ms, "timing": st, "dtype": "f32",
        "config": {"workload": "moe_topk_softmax_align (router + alignment) fp32 [16384, 64] k=6 block 64 seed 1",
                   "padded_len": l_pad, "algorithmic_bytes": bytes_},
        "two_separate_calls": {"ms_per_step": ms_two, "value": bytes_ / ms_two / 1e6, "unit": "GB/s"},
        "graph_replay": None if graph_ms is None else {
            "calls_per_graph": calls, "ms_per_call": ms_gpu, "value": bytes_ / ms_gpu / 1e6,
            "unit": "GB/s",
            "one_call_per_graph_ms": graph1_ms},
        "roofline": {"kernel": "moe_topk_softmax_count_kernel + align_place_fused_kernel (the two "
                               "kernels of one call; GPU time per call from a graph of 20 calls)",
                     "bound": "hbm", "achieved": bytes_ / ms_gpu / 1e6, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": bytes_ / ms_gpu / 1e6 / PEAK_HBM_GBS,
                     "traffic": _traffic("moe_gating"),
                     "note": "5.8 MB working set: launch-latency bound, served from cache"},
    }
    if cpu:
        from oracle import moe_gating as og

        def cpu_step():
            w, ids = og.topk_softmax(logits_cpu, K)
            og.align_block_size(ids, BLK, E)

        dt = _cpu_time(cpu_step)
        res["cpu_baseline"] = {"value": bytes_ / dt / 1e9, "unit": "GB/s",
                               **_cpu_info(), "kind": "port",
                               "sample": "full workload, 1 warm-up + median of 3 reps"}
    return res


def wl_prefill(dev, steps, warmup, cpu):
    from dlcompiler_amd.kernels.prefill_attention import context_attention_fwd

    g = _gen(2)
    lens = torch.randint(512, 4097, (8,), generator=g)
    cu = torch.zeros(9, dtype=torch.int32)
    cu[1:] = lens.cumsum(0)
    total = int(cu[-1])
    q_cpu = torch.randn((total, 32, 128), generator=g).bfloat16()
    k_cpu = torch.randn((total, 8, 128), generator=g).bfloat16()
    v_cpu = torch.randn((total, 8, 128), generator=g).bfloat16()
    q, k, v = q_cpu.to(dev), k_cpu.to(dev), v_cpu.to(dev)
    o = torch.empty_like(q)
    start, seqlen = cu[:-1].to(dev), (cu[1:] - cu[:-1]).to(dev)
    max_len = int(lens.max())
    flops = 4 * 128 * 32 * sum(int(l) * (int(l) + 1) // 2 for l in lens)

    ms, st = _time_steps(
        lambda i: context_attention_fwd(q, k, v, o, start, seqlen, max_len), steps, warmup)
    ms_kernel = st["median_ms"]
    res = {
        "metric": "prefill attention TFLOP/s", "unit": "TFLOP/s", "value": flops / ms / 1e9,
        "ms_per_step": ms, "timing": st, "dtype": "bf16",
        "config": {"workload": "context_attention_fwd causal varlen, 8 seqs U[512,4096] seed 2, "
                               "32q/8kv heads, d128, bf16", "total_tokens": total,
                   "algorithmic_flops": flops},
        "roofline": {"kernel": "prefill_attn_kernel", "bound": "mfma",
                     "achieved": flops / ms_kernel / 1e9, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / ms_kernel / 1e9 / PEAK_BF16_TFLOPS,
                     "traffic": _traffic("prefill_attn")},
    }
    if cpu:
        from oracle import attention as oa

        L = 1024  # one 1024-token sequence, all heads
        qs, ks, vs = q_cpu[:L], k_cpu[:L], v_cpu[:L]
        dt = _cpu_time(lambda: oa.prefill_attention(qs, ks, vs, torch.tensor([0]), torch.tensor([L])))
        sflops = 4 * 128 * 32 * L * (L + 1) // 2
        res["cpu_baseline"] = {"value": sflops / dt / 1e12, "unit": "TFLOP/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"one {L}-token sequence, 32 heads, 1 warm-up + median of 3 reps"}
    return res


def wl_decode(dev, steps, warmup, cpu):
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    g = _gen(3)
    B, HQ, HKV, D, PAGE = 64, 32, 8, 128, 64
    ctx = torch.randint(512, 8193, (B,), generator=g)
    blocks = (ctx + PAGE - 1) // PAGE
    num_pages = int(blocks.sum())
    perm = torch.randperm(num_pages, generator=g).to(torch.int32)
    table = torch.zeros((B, 128), dtype=torch.int32)
    at = 0
    for b in range(B):
        table[b, :blocks[b]] = perm[at:at + blocks[b]]
        at += int(blocks[b])
    kc_cpu = torch.randn((num_pages, PAGE, HKV, D), generator=g).bfloat16()
    vc_cpu = torch.randn((num_pages, PAGE, HKV, D), generator=g).bfloat16()
    q_cpu = torch.randn((B, HQ, D), generator=g).bfloat16()
    nbuf = 2  # two cache copies: 2 x 1.1 GB, well past the 256 MB last-level cache
    kcs = [kc_cpu.to(dev) for _ in range(nbuf)]
    vcs = [vc_cpu.to(dev) for _ in range(nbuf)]
    q, o = q_cpu.to(dev), torch.empty((B, HQ, D), dtype=torch.bfloat16, device=dev)
    table_d, ctx_d = table.to(dev), ctx.to(torch.int32).to(dev)
    ones = torch.ones(B, dtype=torch.int32, device=dev)
    sum_ctx = int(ctx.sum())
    bytes_ = sum_ctx * HKV * D * 2 * 2 + 2 * B * HQ * D * 2 + table.numel() * 4 + B * 4
    flops = 4 * D * HQ * sum_ctx

    def step(i):
        paged_attention_fwd(q, kcs[i % nbuf], vcs[i % nbuf], o, table_d, None, ones, ctx_d, 1)

    ms, st = _time_steps(step, steps, warmup)
    ms_kernel = st["median_ms"]
    # the same step with the index tensors as lmdeploy hands them over (int64): read as they are
    table64, ctx64 = table_d.long(), ctx_d.long()
    ms64, _ = _time_steps(lambda i: paged_attention_fwd(q, kcs[i % nbuf], vcs[i % nbuf], o, table64,
                                                        None, ones, ctx64, 1), steps, warmup)
    res = {
        "metric": "paged decode attention HBM GB/s", "unit": "GB/s", "value": bytes_ / ms / 1e6,
        "ms_per_step": ms, "timing": st, "dtype": "bf16", "tflops": flops / ms / 1e9,
        "int64_index_tensors": {"ms_per_step": ms64, "value": bytes_ / ms64 / 1e6, "unit": "GB/s"},
        "config": {"workload": "paged_attention_fwd decode, batch 64, ctx U[512,8192] seed 3, "
                               "64-token pages, 32q/8kv heads, d128, bf16",
                   "sum_ctx": sum_ctx, "algorithmic_bytes": bytes_},
        "roofline": {"kernel": "paged_decode_split_kernel (+combine)", "bound": "hbm",
                     "achieved": bytes_ / ms_kernel / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": bytes_ / ms_kernel / 1e6 / PEAK_HBM_GBS,
                     "traffic": _traffic("paged_decode")},
    }
    if cpu:
        from oracle import attention as oa

        n = 8
        dt = _cpu_time(lambda: oa.paged_decode(q_cpu[:n], kc_cpu, vc_cpu, table[:n], ctx[:n]),
                       warm=lambda: oa.paged_decode(q_cpu[:1], kc_cpu, vc_cpu, table[:1], ctx[:1]))
        sbytes = int(ctx[:n].sum()) * HKV * D * 4
        res["cpu_baseline"] = {"value": sbytes / dt / 1e9, "unit": "GB/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"first {n} of {B} sequences, 1 warm-up + median of 3 reps"}
    return res


def wl_moe_fp8(dev, steps, warmup, cpu):
    from dlcompiler_amd import _lib
    from dlcompiler_amd.kernels import fused_moe as fm
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size, moe_topk_softmax_align
    from oracle import fp8 as ofp8
    from oracle import moe_gating as og

    T, H, I, E, K = 4096, 2048, 1408, 64, 6
    g = _gen(5)
    x_cpu = torch.randn((T, H), generator=g).bfloat16()
    logits = torch.randn((T, E), generator=g)
    tw_cpu, ids_cpu = og.topk_softmax(logits, K)   # input preparation, untimed
    w1q = torch.empty((E, 2 * I, H), dtype=torch.float8_e4m3fn)
    w1s = torch.empty((E, 2 * I // 128, H // 128))
    w2q = torch.empty((E, H, I), dtype=torch.float8_e4m3fn)
    w2s = torch.empty((E, H // 128, I // 128))
    for e in range(E):  # offline weight quantisation (input preparation, untimed)
        w1q[e], w1s[e] = ofp8.block_quant_weight(torch.randn((2 * I, H), generator=g) * 0.02)
        w2q[e], w2s[e] = ofp8.block_quant_weight(torch.randn((H, I), generator=g) * 0.02)
    x, tw, ids = x_cpu.to(dev), tw_cpu.to(dev), ids_cpu.to(dev)
    plain = [t.to(dev) for t in (w1q, w1s, w2q, w2s)]
    # operand order: the weights re-arranged once at load time (untimed, like the quantisation)
    shuf = [fm.shuffle_moe_weight_fp8(plain[0]), plain[1], fm.shuffle_moe_weight_fp8(plain[2]), plain[3]]
    flops = 2 * T * K * H * 2 * I + 2 * T * K * I * H
    gate_up_flops, down_flops = 2 * T * K * H * 2 * I, 2 * T * K * I * H

    def kernel_times(dw, shuffled):
        """Median duration of the two grouped-GEMM launches, each timed alone on the inputs the
        step gives it (events around batches of launches of that one kernel)."""
        lib = _lib.load()
        block = fm._BLOCK_M
        sorted_ids, _, _, counts = moe_align_block_size(ids, block, E, return_counts=True)
        nmb = sorted_ids.numel() // block
        xq, xs = fm.per_token_group_quant_fp8(x)
        hq = torch.empty((nmb * block, I), dtype=torch.float8_e4m3fn, device=dev)
        hs = torch.empty((nmb * block, I // 128), dtype=torch.float32, device=dev)
        slots = torch.empty((T * K, H), dtype=torch.bfloat16, device=dev)
        stream = _lib.current_stream_ptr(dev)

        def gate_up(i):
            _lib.check(lib.dlb_moe_gemm_fp8_gate_up(
                xq.data_ptr(), xs.data_ptr(), dw[0].data_ptr(), dw[1].data_ptr(), sorted_ids.data_ptr(),
                counts.data_ptr(), E, nmb, block, T, K, H, I, 0, E, int(shuffled), hq.data_ptr(),
                hs.data_ptr(), stream), "gate_up")

        def down(i):
            _lib.check(lib.dlb_moe_gemm_fp8_down(
                hq.data_ptr(), hs.data_ptr(), dw[2].data_ptr(), dw[3].data_ptr(), sorted_ids.data_ptr(),
                counts.data_ptr(), E, tw.data_ptr(), nmb, block, T, K, H, I, 0, E, int(shuffled),
                slots.data_ptr(), 0, stream), "down")

        for i in range(MIN_WARMUP):
            gate_up(i)
            down(i)
        return _batch_stats(gate_up), _batch_stats(down)

    layouts = {}
    for name, dw, shuffled in (("operand-order", shuf, True), ("row-major", plain, False)):
        ms, st = _time_steps(lambda i: fm.fused_moe_fp8(x, *dw, tw, ids, K, weights_shuffled=shuffled),
                             steps, warmup)
        graph_ms = _graph_replay_ms(
            lambda: fm.fused_moe_fp8(x, *dw, tw, ids, K, weights_shuffled=shuffled), 20, 5, "moe " + name)
        st_gu, st_dn = kernel_times(dw, shuffled)
        # the same step when the layer's router has already produced the expert alignment
        # (moe_topk_softmax_align) and hands it over: the routing is sorted once per layer
        al_sorted, _, _, al_counts = moe_align_block_size(ids, fm.ALIGN_BLOCK, E, return_counts=True)
        ms_al, _ = _time_steps(lambda i: fm.fused_moe_fp8(x, *dw, tw, ids, K, weights_shuffled=shuffled,
                                                         alignment=(al_sorted, al_counts)), steps, warmup)
        # and the whole layer from the router's logits: softmax + top-k + alignment (one native call
        # of two launches), then the MLP on the alignment that call returns
        logits_dev = logits.to(dev)

        def from_logits(i):
            w_, ids_, so_, _, _, cn_ = moe_topk_softmax_align(logits_dev, K, fm.ALIGN_BLOCK,
                                                                 return_counts=True)
            fm.fused_moe_fp8(x, *dw, w_, ids_, K, weights_shuffled=shuffled, alignment=(so_, cn_))

        ms_fl, _ = _time_steps(from_logits, steps, warmup)
        layouts[name] = {
            "ms_per_step": ms, "value": flops / ms / 1e9, "unit": "TFLOP/s", "timing": st,
            "graph_replay_ms": graph_ms,
            "alignment_handed_over": {"ms_per_step": ms_al, "value": flops / ms_al / 1e9, "unit": "TFLOP/s"},
            "from_router_logits": {"ms_per_step": ms_fl, "value": flops / ms_fl / 1e9, "unit": "TFLOP/s",
                                   "note": "router softmax + top-k + alignment included in the step"},
            "gate_up_kernel": dict(st_gu, tflops=gate_up_flops / st_gu["median_ms"] / 1e9,
                                   frac=gate_up_flops / st_gu["median_ms"] / 1e9 / PEAK_FP8_TFLOPS),
            "down_kernel": dict(st_dn, tflops=down_flops / st_dn["median_ms"] / 1e9,
                                frac=down_flops / st_dn["median_ms"] / 1e9 / PEAK_FP8_TFLOPS),
        }
    best = layouts["operand-order"]
    ms = best["ms_per_step"]
    ms_gate_up = best["gate_up_kernel"]["median_ms"]
    res = {
        "metric": "fp8 fused-MoE TFLOP/s", "unit": "TFLOP/s", "value": flops / ms / 1e9,
        "ms_per_step": ms, "timing": best["timing"], "dtype": "fp8_e4m3",
        "config": {"workload": "fused_moe_fp8 T=4096 H=2048 I=1408 E=64 top-6, fp8 e4m3 weights "
                               "128x128 block scales, per-token-group act quant, seed 5",
                   "weight_layout": "operand-order (re-arranged once at load time; the reference's "
                                    "row-major layout is under weight_layouts)",
                   "algorithmic_flops": flops},
        "weight_layouts": layouts,
        "gemm_only_tflops": flops / (ms_gate_up + best["down_kernel"]["median_ms"]) / 1e9,
        "roofline": {"kernel": "moe_gemm_kernel<gate_up>", "bound": "mfma",
                     "achieved": gate_up_flops / ms_gate_up / 1e9, "peak": PEAK_FP8_TFLOPS,
                     "unit": "TFLOP/s", "frac": gate_up_flops / ms_gate_up / 1e9 / PEAK_FP8_TFLOPS,
                     "traffic": _traffic("moe_gemm_fp8_gate_up")},
    }
    if cpu:
        from oracle import fused_moe as ofm

        # the whole workload, repeated: about ten seconds of CPU work on the box's 16 cores
        ofm.fused_moe_fp8(x_cpu[:64], w1q, w1s, w2q, w2s, tw_cpu[:64], ids_cpu[:64])  # warm-up
        reps = 0
        t0 = time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10.0 and reps < 40):
            ofm.fused_moe_fp8(x_cpu, w1q, w1s, w2q, w2s, tw_cpu, ids_cpu)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": flops / dt / 1e12, "unit": "TFLOP/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"all {T} tokens, {reps} reps ({dt * reps:.1f} s of CPU time)"}
    return res


def wl_moe_bf16(dev, steps, warmup, cpu):
    """The reference's own fused_moe (python/dlBLAS/dlblas/kernels/fused_moe.py:296-376) at the
    config-5 shape in bf16: 4096 tokens, hidden 2048, intermediate 1408, 64 experts, top-6."""
    from dlcompiler_amd import _lib
    from dlcompiler_amd.kernels import fused_moe as fm
    from dlcompiler_amd.kernels.moe_gating import moe_align_block_size
    from oracle import moe_gating as og

    T, H, I, E, K = 4096, 2048, 1408, 64, 6
    g = _gen(5)
    x_cpu = torch.randn((T, H), generator=g).bfloat16()
    logits = torch.randn((T, E), generator=g)
    tw_cpu, ids_cpu = og.topk_softmax(logits, K)   # input preparation, untimed
    w1_cpu = torch.empty((E, 2 * I, H), dtype=torch.bfloat16)
    w2_cpu = torch.empty((E, H, I), dtype=torch.bfloat16)
    for e in range(E):
        w1_cpu[e] = (torch.randn((2 * I, H), generator=g) * 0.02).bfloat16()
        w2_cpu[e] = (torch.randn((H, I), generator=g) * 0.02).bfloat16()
    x, tw, ids = x_cpu.to(dev), tw_cpu.to(dev), ids_cpu.to(dev)
    plain = [w1_cpu.to(dev), w2_cpu.to(dev)]
    shuf = [fm.shuffle_moe_weight(plain[0]), fm.shuffle_moe_weight(plain[1])]
    gate_up_flops, down_flops = 2 * T * K * H * 2 * I, 2 * T * K * I * H
    flops = gate_up_flops + down_flops

    def kernel_times(dw, shuffled):
        lib = _lib.load()
        block = fm._BLOCK_M
        sorted_ids, _, _, counts = moe_align_block_size(ids, block, E, return_counts=True)
        nmb = sorted_ids.numel() // block
        act = torch.empty((nmb * block, I), dtype=torch.bfloat16, device=dev)
        slots = torch.empty((T * K, H), dtype=torch.bfloat16, device=dev)
        stream = _lib.current_stream_ptr(dev)

        def gate_up(i):
            _lib.check(lib.dlb_moe_gemm_16bit_gate_up(
                x.data_ptr(), dw[0].data_ptr(), sorted_ids.data_ptr(), counts.data_ptr(), E, nmb, block,
                T, K, H, I, 0, E, int(shuffled), act.data_ptr(), 0, stream), "gate_up")

        def down(i):
            _lib.check(lib.dlb_moe_gemm_16bit_down(
                act.data_ptr(), dw[1].data_ptr(), sorted_ids.data_ptr(), counts.data_ptr(), E,
                tw.data_ptr(), nmb, block, T, K, H, I, 0, E, int(shuffled), slots.data_ptr(), 0,
                stream), "down")

        for i in range(MIN_WARMUP):
            gate_up(i)
            down(i)
        return _batch_stats(gate_up), _batch_stats(down)

    layouts = {}
    for name, dw, shuffled in (("row-major", plain, False), ("operand-order", shuf, True)):
        ms, st = _time_steps(lambda i: fm.fused_moe(x, *dw, tw, ids, K, weights_shuffled=shuffled),
                             steps, warmup)
        st_gu, st_dn = kernel_times(dw, shuffled)
        layouts[name] = {
            "ms_per_step": ms, "value": flops / ms / 1e9, "unit": "TFLOP/s", "timing": st,
            "gate_up_kernel": dict(st_gu, tflops=gate_up_flops / st_gu["median_ms"] / 1e9,
                                   frac=gate_up_flops / st_gu["median_ms"] / 1e9 / PEAK_BF16_TFLOPS),
            "down_kernel": dict(st_dn, tflops=down_flops / st_dn["median_ms"] / 1e9,
                                frac=down_flops / st_dn["median_ms"] / 1e9 / PEAK_BF16_TFLOPS),
        }
    # the reference's signature and weight layout are the figure of this workload
    ref_l = layouts["row-major"]
    ms = ref_l["ms_per_step"]
    ms_gate_up = ref_l["gate_up_kernel"]["median_ms"]
    res = {
        "metric": "bf16 fused-MoE TFLOP/s", "unit": "TFLOP/s", "value": flops / ms / 1e9,
        "ms_per_step": ms, "timing": ref_l["timing"], "dtype": "bf16",
        "config": {"workload": "fused_moe T=4096 H=2048 I=1408 E=64 top-6, bf16 weights in the "
                               "reference's row-major [E, N, K] layout, seed 5",
                   "algorithmic_flops": flops},
        "weight_layouts": layouts,
        "roofline": {"kernel": "moe_gemm_kernel<gate_up, bf16>", "bound": "mfma",
                     "achieved": gate_up_flops / ms_gate_up / 1e9, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": gate_up_flops / ms_gate_up / 1e9 / PEAK_BF16_TFLOPS,
                     "traffic": _traffic("moe_gemm_bf16_gate_up")},
    }
    if cpu:
        from oracle import fused_moe as ofm

        n = 1024   # a quarter of the tokens against all experts
        dt = _cpu_time(lambda: ofm.fused_moe(x_cpu[:n], w1_cpu, w2_cpu, tw_cpu[:n], ids_cpu[:n]),
                       warm=lambda: ofm.fused_moe(x_cpu[:64], w1_cpu, w2_cpu, tw_cpu[:64], ids_cpu[:64]))
        res["cpu_baseline"] = {"value": flops * n / T / dt / 1e12, "unit": "TFLOP/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"first {n} of {T} tokens, 1 warm-up + median of 3 reps"}
    return res


def _hbm_result(metric, workload, bytes_, ms, st, kernel, dtype="bf16", traffic=None):
    ms_kernel = st["median_ms"]
    return {
        "metric": metric, "unit": "GB/s", "value": bytes_ / ms / 1e6, "ms_per_step": ms,
        "timing": st,
        "dtype": dtype, "config": {"workload": workload, "algorithmic_bytes": bytes_},
        "roofline": {"kernel": kernel, "bound": "hbm", "achieved": bytes_ / ms_kernel / 1e6,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": bytes_ / ms_kernel / 1e6 / PEAK_HBM_GBS, "traffic": _traffic(traffic)},
    }


def wl_add_rms_norm(dev, steps, warmup, cpu):
    """Decoder-layer neighbour: residual add + RMSNorm, [16384, 4096] bf16 (read x, residual;
    write out, new residual; the weight row is noise)."""
    from dlcompiler_amd.kernels.rms_norm import rms_norm

    M, N, nbuf = 16384, 4096, 3
    g = _gen(6)
    xs = [torch.randn((M, N), generator=g).bfloat16().to(dev) for _ in range(nbuf)]
    rs = [torch.randn((M, N), generator=g).bfloat16().to(dev) for _ in range(nbuf)]
    w = torch.randn((N,), generator=g).bfloat16().to(dev)
    outs = [torch.empty_like(xs[0]) for _ in range(nbuf)]
    ors = [torch.empty_like(xs[0]) for _ in range(nbuf)]
    bytes_ = 4 * M * N * 2 + N * 2
    ms, msk = _time_steps(lambda i: rms_norm(xs[i % nbuf], w, 1e-6, residual=rs[i % nbuf],
                                             out=outs[i % nbuf], out_residual=ors[i % nbuf]),
                          steps, warmup)
    res = _hbm_result("add_rms_norm HBM GB/s", "rms_norm with residual, bf16 [16384, 4096] seed 6",
                      bytes_, ms, msk, "rms_norm_kernel<add>", traffic="add_rms_norm")
    if cpu:
        from oracle import decoder_ops as od

        x, r, wc = xs[0][:2048].cpu(), rs[0][:2048].cpu(), w.cpu()
        dt = _cpu_time(lambda: od.rms_norm(x, wc, 1e-6, residual=r))
        res["cpu_baseline"] = {"value": bytes_ * 2048 / M / dt / 1e9, "unit": "GB/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"2048 of {M} rows, 1 warm-up + median of 3 reps"}
    return res


def wl_rotary(dev, steps, warmup, cpu):
    """Decoder-layer neighbour: rotary embedding of q [16384, 32, 128] and k [16384, 8, 128]."""
    from dlcompiler_amd.kernels.apply_rotary_pos_emb import apply_rotary_pos_emb

    T, HQ, HK, D, nbuf = 16384, 32, 8, 128, 3
    g = _gen(7)
    qs = [torch.randn((T, HQ, D), generator=g).bfloat16().to(dev) for _ in range(nbuf)]
    ks = [torch.randn((T, HK, D), generator=g).bfloat16().to(dev) for _ in range(nbuf)]
    ang = torch.rand((T, D // 2), generator=g) * 6.28
    cos = torch.cat([ang.cos(), ang.cos()], -1).bfloat16().to(dev)
    sin = torch.cat([ang.sin(), ang.sin()], -1).bfloat16().to(dev)
    qo = [torch.empty_like(qs[0]) for _ in range(nbuf)]
    ko = [torch.empty_like(ks[0]) for _ in range(nbuf)]
    bytes_ = 2 * T * (HQ + HK) * D * 2 + 2 * T * D * 2
    ms, msk = _time_steps(lambda i: apply_rotary_pos_emb(qs[i % nbuf], ks[i % nbuf], cos, sin,
                                                         qo[i % nbuf], ko[i % nbuf]), steps, warmup)
    res = _hbm_result("apply_rotary_pos_emb HBM GB/s",
                      "apply_rotary_pos_emb bf16 q [16384, 32, 128], k [16384, 8, 128] seed 7",
                      bytes_, ms, msk, "rotary_kernel", traffic="apply_rotary_pos_emb")
    if cpu:
        from oracle import decoder_ops as od

        n = 2048
        cq, ck, cc, cs_ = qs[0][:n].cpu(), ks[0][:n].cpu(), cos[:n, None].cpu(), sin[:n, None].cpu()
        dt = _cpu_time(lambda: od.apply_rotary_pos_emb(cq, ck, cc, cs_))
        res["cpu_baseline"] = {"value": bytes_ * n / T / dt / 1e9, "unit": "GB/s",
                               **_cpu_info(), "kind": "port",
                               "sample": f"{n} of {T} tokens, 1 warm-up + median of 3 reps"}
    return res


def wl_fill_kv_cache(dev, steps, warmup, cpu):
    """The step before attention: scatter the new K/V rows of a prefill batch (config-3
    lengths) into 64-token pages, 8 KV heads, d128."""
    from dlcompiler_amd.kernels.fill_kv_cache import fill_kv_cache

    g = _gen(2)
    B, HKV, D, PAGE = 8, 8, 128, 64
    lens = torch.randint(512, 4097, (B,), generator=g)
    T = int(lens.sum())
    blocks = (lens + PAGE - 1) // PAGE
    num_pages = int(blocks.sum())
    perm = torch.randperm(num_pages, generator=g).to(torch.int32)
    table = torch.zeros((B, int(blocks.max())), dtype=torch.int32)
    at = 0
    for b in range(B):
        table[b, :blocks[b]] = perm[at:at + blocks[b]]
        at += int(blocks[b])
    nbuf = 2
    k = [torch.randn((T, HKV, D), generator=g).bfloat16().to(dev) for _ in range(nbuf)]
    v = [torch.randn((T, HKV, D), generator=g).bfloat16().to(dev) for _ in range(nbuf)]
    kc = [torch.zeros((num_pages, PAGE, HKV, D), dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
    vc = [torch.zeros((num_pages, PAGE, HKV, D), dtype=torch.bfloat16, device=dev) for _ in range(nbuf)]
    start = (torch.cumsum(lens, 0) - lens).to(torch.int32).to(dev)
    lens_d, table_d = lens.to(torch.int32).to(dev), table.to(dev)
    bytes_ = 4 * T * HKV * D * 2
    ms, msk = _time_steps(lambda i: fill_kv_cache(k[i % nbuf], v[i % nbuf], kc[i % nbuf], vc[i % nbuf],
                                                  start, lens_d, lens_d, int(lens.max()), table_d),
                          steps, warmup)
    res = _hbm_result("fill_kv_cache HBM GB/s",
                      f"fill_kv_cache bf16, 8 seqs U[512,4096] seed 2 ({T} tokens), 8 kv heads, d128, 64-token pages",
                      bytes_, ms, msk, "fill_kv_cache_kernel", traffic="fill_kv_cache")
    if cpu:
        from oracle import decoder_ops as od

        l0 = int(lens[0])
        ck, cv, ckc, cvc = k[0][:l0].cpu(), v[0][:l0].cpu(), kc[0].cpu(), vc[0].cpu()
        dt = _cpu_time(lambda: od.fill_kv_cache(ck, cv, ckc, cvc, [l0], [0], table[:1]))
        res["cpu_baseline"] = {"value": bytes_ * l0 / T / dt / 1e9, "unit": "GB/s",
                               **_cpu_info(1), "kind": "port",
                               "sample": f"first sequence ({l0} tokens), 1 warm-up + median of 3 reps "
                                         "(each includes the oracle's copy of the cache)"}
    return res


def wl_paged_prefill(dev, steps, warmup, cpu):
    """Chunked prefill: 8 sequences, 512 new tokens each after a history U[512, 4096] already in
    the paged cache (paged_attention_fwd, non-decoding branch)."""
    from dlcompiler_amd.kernels.paged_attention import paged_attention_fwd

    g = _gen(8)
    B, HQ, HKV, D, PAGE, QL = 8, 32, 8, 128, 64, 512
    hist = torch.randint(512, 4097, (B,), generator=g)
    kvl = hist + QL
    blocks = (kvl + PAGE - 1) // PAGE
    num_pages = int(blocks.sum())
    perm = torch.randperm(num_pages, generator=g).to(torch.int32)
    table = torch.zeros((B, int(blocks.max())), dtype=torch.int32)
    at = 0
    for b in range(B):
        table[b, :blocks[b]] = perm[at:at + blocks[b]]
        at += int(blocks[b])
    kc = torch.randn((num_pages, PAGE, HKV, D), generator=g).bfloat16().to(dev)
    vc = torch.randn((num_pages, PAGE, HKV, D), generator=g).bfloat16().to(dev)
    q = torch.randn((B * QL, HQ, D), generator=g).bfloat16().to(dev)
    o = torch.empty_like(q)
    start = (torch.arange(B) * QL).to(torch.int32).to(dev)
    ql = torch.full((B,), QL, dtype=torch.int32, device=dev)
    kvl_d, table_d = kvl.to(torch.int32).to(dev), table.to(dev)
    pairs = sum(QL * int(h) + QL * (QL + 1) // 2 for h in hist)
    flops = 4 * D * HQ * pairs
    ms, st = _time_steps(lambda i: paged_attention_fwd(q, kc, vc, o, table_d, start, ql, kvl_d, QL),
                         steps, warmup)
    msk = st["median_ms"]
    res = {
        "metric": "paged prefill attention TFLOP/s", "unit": "TFLOP/s", "value": flops / ms / 1e9,
        "ms_per_step": ms, "timing": st, "dtype": "bf16",
        "config": {"workload": "paged_attention_fwd prefill, 8 seqs x 512 new tokens after history "
                               "U[512,4096] seed 8, 64-token pages, 32q/8kv heads, d128, bf16",
                   "algorithmic_flops": flops},
        "roofline": {"kernel": "prefill_attn_kernel<paged>", "bound": "mfma",
                     "achieved": flops / msk / 1e9, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / msk / 1e9 / PEAK_BF16_TFLOPS,
                     "traffic": _traffic("paged_prefill")},
    }
    if cpu:
        from oracle import attention as oa

        cq, ckc, cvc = q[:QL].cpu(), kc.cpu(), vc.cpu()
        dt = _cpu_time(lambda: oa.paged_prefill(cq, ckc, cvc, table[:1], torch.tensor([0]),
                                                torch.tensor([QL]), kvl[:1]))
        f1 = 4 * D * HQ * (QL * int(hist[0]) + QL * (QL + 1) // 2)
        res["cpu_baseline"] = {"value": f1 / dt / 1e12, "unit": "TFLOP/s",
                               **_cpu_info(), "kind": "port",
                               "sample": "first sequence, 1 warm-up + median of 3 reps"}
    return res


_probe_lib = None


def load_probe_lib():
    """ctypes binding of ``libdlblas_bench_probe.so`` (``dlcompiler_amd/csrc/bench/bench_probe.h``):
    the two measurement kernels behind ``box``; a library of its own, built with the operators'."""
    global _probe_lib
    if _probe_lib is None:
        import ctypes
        from ctypes import c_int, c_int64, c_void_p

        from dlcompiler_amd.build import PROBE_LIB_PATH

        if not PROBE_LIB_PATH.exists():
            raise ImportError(f"{PROBE_LIB_PATH} not found: build it with `python -m dlcompiler_amd.build`")
        lib = ctypes.CDLL(str(PROBE_LIB_PATH))
        lib.dlb_probe_mfma_operand_bytes.restype = c_int64
        lib.dlb_probe_mfma_operand_bytes.argtypes = [c_int]
        lib.dlb_probe_mfma_rate.restype = c_int
        lib.dlb_probe_mfma_rate.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                            c_void_p]
        lib.dlb_probe_hbm_read.restype = c_int
        lib.dlb_probe_hbm_read.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p]
        _probe_lib = lib
    return _probe_lib


def measure_box(dev):
    """What this chip sustains, measured in this run: the matrix-instruction rate on random and on
    all-zero operands (the clock under matrix load follows the power the operand data draws, so
    the two differ by a third; the published peaks correspond to the all-zero case) and the rate
    of a plain non-temporal stream.  Reported beside every roofline, never instead of it."""
    from dlcompiler_amd import _lib

    lib = load_probe_lib()
    blocks = torch.cuda.get_device_properties(dev).multi_processor_count
    nbytes = lib.dlb_probe_mfma_operand_bytes(blocks)
    sink = torch.zeros(512, dtype=torch.float32, device=dev)
    sink_bytes = sink.numel() * 4
    stream = _lib.current_stream_ptr(dev)
    g = _gen(99)
    n16 = nbytes // 2
    operands = {
        "bf16_randn": torch.randn(n16, generator=g).bfloat16().to(dev),
        "bf16_zeros": torch.zeros(n16, dtype=torch.bfloat16, device=dev),
        "fp8_randn": torch.randn(nbytes, generator=g).to(torch.float8_e4m3fn).to(dev),
        "fp8_zeros": torch.zeros(nbytes, dtype=torch.uint8, device=dev),
    }
    out = {}

    def mfma_rate(buf, fp8, valu):
        iters = 20000 if fp8 else 40000   # about 12 ms per launch on random operands

        def launch():
            _lib.check(lib.dlb_probe_mfma_rate(buf.data_ptr(), nbytes, sink.data_ptr(), sink_bytes,
                                               blocks, fp8, iters, valu, stream), "dlb_probe_mfma_rate")

        for _ in range(3):
            launch()
        torch.cuda.synchronize()
        t = Timer()
        ev = t.start()
        for _ in range(3):
            launch()
        t.stop(ev)
        ms = t.mean_ms() / 3
        return blocks * 8 * iters * 4 * (131072 if fp8 else 32768) / ms / 1e9

    for key, buf in operands.items():
        out[f"mfma_{key}_tflops"] = mfma_rate(buf, int(key.startswith("fp8")), 0)
    # the same stream with 8 independent fp32 multiply-adds of the wave behind every MFMA: what
    # the SIMD hides of a wave's vector arithmetic under its matrix instructions (the prefill
    # kernel issues about 5 vector instructions per bf16 MFMA, 32 of them exponentials per tile;
    # the fp8 GEMM's main loop about 10 per MFMA, 8 of them the block-scale multiplies)
    out["mfma_bf16_randn_valu8_tflops"] = mfma_rate(operands["bf16_randn"], 0, 8)
    out["mfma_fp8_randn_valu8_tflops"] = mfma_rate(operands["fp8_randn"], 1, 8)
    x = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()   # 1 GiB
    nb = x.numel() * 4

    def read():
        _lib.check(lib.dlb_probe_hbm_read(x.data_ptr(), sink.data_ptr(), sink_bytes, nb, stream),
                   "dlb_probe_hbm_read")

    for _ in range(3):
        read()
    torch.cuda.synchronize()
    t = Timer()
    ev = t.start()
    for _ in range(10):
        read()
    t.stop(ev)
    out["hbm_read_gbs"] = nb / (t.mean_ms() / 10) / 1e6
    out["note"] = ("measured in this run: back-to-back MFMAs (bf16 32x32x16 / fp8 32x32x64, two waves "
                   "per SIMD on every CU, nothing else in the loop) on random-normal and on all-zero "
                   "operands; valu8: the same with 8 independent fp32 multiply-adds of the wave after "
                   "every MFMA; a read-only non-temporal stream over 1 GiB")
    del x
    torch.cuda.empty_cache()
    return out


def _add_measured_ceiling(res, box):
    """roofline.measured_peak / frac_of_measured: the same achieved figure against what the chip
    sustained in this run on random operands (MFMA-bound) or in a read-only stream (HBM-bound)."""
    rf = res["roofline"]
    if rf["bound"] == "mfma":
        peak = box["mfma_fp8_randn_tflops"] if rf["peak"] == PEAK_FP8_TFLOPS else box["mfma_bf16_randn_tflops"]
    else:
        peak = box["hbm_read_gbs"]
    rf["measured_peak"] = peak
    rf["frac_of_measured"] = rf["achieved"] / peak


WORKLOADS = {
    "silu_and_mul": wl_silu,
    "moe_gating": wl_gating,
    "prefill_attention": wl_prefill,
    "paged_decode": wl_decode,
    "moe_fp8": wl_moe_fp8,
    # the reference's own fused_moe (bf16) at the same shape
    "moe_bf16": wl_moe_bf16,
    # the neighbours of the five configurations in a decoder layer
    "add_rms_norm": wl_add_rms_norm,
    "apply_rotary_pos_emb": wl_rotary,
    "fill_kv_cache": wl_fill_kv_cache,
    "paged_prefill": wl_paged_prefill,
}
PRIMARY = "moe_fp8"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=["all", *WORKLOADS])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first launch an elementwise copy of 1 GiB (fp32 x * 1 -> y) three times: "
                         "the known-size kernel that scales rocprofv3's FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--counters", action="store_true",
                    help="for a run under rocprofv3 --pmc, where every launch is serialised: "
                         "--warmup is taken as given, 4 statistics iterations instead of "
                         f"{STAT_ITERS}, no graph replays; the timings of such a run mean nothing")
    args = ap.parse_args()
    global COUNTER_PASS
    COUNTER_PASS = args.counters
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the operators are single-device; "
              "no collective is part of the path) -- run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from dlcompiler_amd import _lib

    _lib.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        x = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        y = torch.empty_like(x)
        for _ in range(3):
            torch.mul(x, 1.0, out=y)
        torch.cuda.synchronize()
        del x, y
        torch.cuda.empty_cache()
    box = None if args.counters else measure_box(dev)
    if box is not None:
        print("[bench] this chip, measured: MFMA bf16 %.0f TFLOP/s on random operands (%.0f on zeros, %.0f "
              "with 8 vector multiply-adds per MFMA), fp8 %.0f (%.0f, %.0f), read-only HBM stream %.0f GB/s" % (
                  box["mfma_bf16_randn_tflops"], box["mfma_bf16_zeros_tflops"],
                  box["mfma_bf16_randn_valu8_tflops"],
                  box["mfma_fp8_randn_tflops"], box["mfma_fp8_zeros_tflops"],
                  box["mfma_fp8_randn_valu8_tflops"], box["hbm_read_gbs"]),
              file=sys.stderr, flush=True)
    names = list(WORKLOADS) if args.workload == "all" else [args.workload]
    primary = PRIMARY if args.workload == "all" else args.workload
    results = {}
    for name in names:
        t0 = time.perf_counter()
        results[name] = WORKLOADS[name](dev, args.steps, args.warmup, not args.no_cpu)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        if box is not None:
            _add_measured_ceiling(results[name], box)
        print(f"[bench] {name}: {results[name]['value']:.2f} {results[name]['unit']} "
              f"({results[name]['ms_per_step'] * 1e3:.1f} us/step, roofline "
              f"{results[name]['roofline']['frac'] * 100:.1f}%) in {time.perf_counter() - t0:.1f}s",
              file=sys.stderr, flush=True)
    p = results[primary]
    line = {
        "metric": p["metric"], "value": p["value"], "unit": p["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": p["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": p["dtype"],
        "data": "synthetic", "config": p["config"], "roofline": p["roofline"],
        "cpu_baseline": p.get("cpu_baseline"),
        "host": {"cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(),
                 "cpu_model": _cpu_model()},
        "box": box,
        "traffic_note": TRAFFIC_NOTE,
        "workloads": results,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
