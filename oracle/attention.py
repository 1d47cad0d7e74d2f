"""Oracle for the attention operators (test infrastructure).

* ``prefill_attention`` restates the ground truth of
  python/dlBLAS/tests/kernels/test_prefill_attention.py:11-36 (dense causal attention per
  sequence: scores / sqrt(D), softmax in fp32, probabilities cast to the input dtype before
  the product with V) for the packed varlen layout and GQA head mapping of
  python/dlBLAS/dlblas/kernels/prefill_attention.py:155-159 (``kv_head = q_head // group``).
* ``paged_decode`` restates python/dlBLAS/tests/kernels/test_paged_attention.py:28-84:
  the paged cache is gathered through the block table into contiguous K/V
  (``_make_blocked_cache`` read backwards), then ``_naive_attention``: GQA expand,
  ``softmax(q k^T / sqrt(D))`` in fp32, cast to the query dtype, ``@ v``.

* ``paged_prefill`` is the same ground truth for new tokens that follow a cached history
  (test_paged_attention.py:15-27 ``_make_bias``: key j is hidden from query i when
  ``j - i > history``), with the sliding window of ``_naive_window_attention`` (:87-113,
  flash-attn ``window_size=(w, w)`` under ``causal=True``: keys ``>= position - w``).

All evaluate the two matrix products with fp32 accumulation on the 16-bit inputs and do not
round the scores to 16 bits (the reference's fp16 matmul on the device does); outputs are
rounded once to the input dtype.
"""
from __future__ import annotations

import math

import torch


def _dense_attention(q, k, v, scale, causal, window=None, softcap=None):
    """q [Hq, Lq, D], k/v [Hkv, Lk, D] -> [Hq, Lq, D] in q.dtype.  The queries are the last
    Lq positions of the Lk keys.  ``window`` > 0 hides keys more than ``window`` positions
    behind a query (python/dlBLAS/dlblas/kernels/paged_attention.py:163-167,191-199);
    ``softcap`` > 0 maps the scaled scores to cap * tanh(scores / cap) (:186-189)."""
    hq, hkv = q.shape[0], k.shape[0]
    group = hq // hkv
    kk = k.float().repeat_interleave(group, dim=0)
    vv = v.float().repeat_interleave(group, dim=0)
    scores = torch.matmul(q.float(), kk.transpose(1, 2)) * scale
    if softcap is not None and softcap > 0:
        scores = torch.tanh(scores / softcap) * softcap
    lq, lk = q.shape[1], k.shape[1]
    if causal:
        keep = torch.ones(lq, lk, dtype=torch.bool).tril(diagonal=lk - lq)
        scores = scores.masked_fill(~keep, float("-inf"))
    if window is not None and window > 0:
        qpos = torch.arange(lk - lq, lk)[:, None]
        far = torch.arange(lk)[None, :] < qpos - window
        scores = scores.masked_fill(far, float("-inf"))
    p = torch.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype)
    return torch.matmul(p.float(), vv).to(q.dtype)


def prefill_attention(q, k, v, b_start_loc, b_seq_len, sm_scale=None):
    """q [T, Hq, D], k/v [T, Hkv, D] packed; returns o [T, Hq, D] (rows outside any
    sequence are left zero)."""
    scale = sm_scale if sm_scale is not None else 1.0 / math.sqrt(q.shape[-1])
    o = torch.zeros_like(q)
    for start, length in zip(b_start_loc.tolist(), b_seq_len.tolist()):
        if length <= 0:
            continue
        sl = slice(start, start + length)
        o[sl] = _dense_attention(q[sl].transpose(0, 1), k[sl].transpose(0, 1),
                                 v[sl].transpose(0, 1), scale, True).transpose(0, 1)
    return o


def gather_paged(cache, block_table_row, length):
    """[pages, page, H, D] -> contiguous [length, H, D] for one sequence."""
    page = cache.shape[1]
    n = -(-length // page)
    pages = cache[block_table_row[:n].long()]
    return pages.reshape(n * page, *cache.shape[2:])[:length]


def paged_decode(q, k_cache, v_cache, block_table, kv_len, sm_scale=None, window=None,
                 softcap=None):
    """q [B, Hq, D] -> o [B, Hq, Dv] (Dv = value head size of the cache); sequences with
    kv_len <= 0 give zeros."""
    scale = sm_scale if sm_scale is not None else 1.0 / math.sqrt(q.shape[-1])
    o = q.new_zeros((*q.shape[:-1], v_cache.shape[-1]))
    for b, length in enumerate(kv_len.tolist()):
        if length <= 0:
            continue
        kk = gather_paged(k_cache, block_table[b], length).transpose(0, 1)
        vv = gather_paged(v_cache, block_table[b], length).transpose(0, 1)
        o[b] = _dense_attention(q[b][:, None, :], kk, vv, scale, False, window, softcap)[:, 0, :]
    return o


def paged_prefill(q, k_cache, v_cache, block_table, q_start_loc, q_len, kv_len, sm_scale=None,
                  window=None, softcap=None):
    """q [T, Hq, D] packed; sequence b owns rows q_start_loc[b] .. + q_len[b], which are the
    last q_len[b] of its kv_len[b] cached positions.  Returns o [T, Hq, Dv]; rows outside any
    sequence stay zero."""
    scale = sm_scale if sm_scale is not None else 1.0 / math.sqrt(q.shape[-1])
    o = q.new_zeros((*q.shape[:-1], v_cache.shape[-1]))
    for b, (start, lq, lk) in enumerate(zip(q_start_loc.tolist(), q_len.tolist(), kv_len.tolist())):
        if lq <= 0 or lk < lq:
            continue
        kk = gather_paged(k_cache, block_table[b], lk).transpose(0, 1)
        vv = gather_paged(v_cache, block_table[b], lk).transpose(0, 1)
        sl = slice(start, start + lq)
        o[sl] = _dense_attention(q[sl].transpose(0, 1), kk, vv, scale, True, window,
                                 softcap).transpose(0, 1)
    return o


def make_paged_cache(k_seqs, v_seqs, page, num_pages=None, seed=0, dtype=None):
    """Scatter per-sequence K ([L_i, H, D]) and V ([L_i, H, Dv]) into a paged cache with pages assigned by
    a seeded random permutation.  Returns (k_cache, v_cache, block_table int32 [B, max_blocks]).
    Unused table slots are 0; unused cache rows hold NaN so that any read past a context shows."""
    lens = [t.shape[0] for t in k_seqs]
    blocks = [-(-l // page) for l in lens]
    total = sum(blocks)
    num_pages = num_pages or max(total, 1)
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g)[:total].to(torch.int32)
    h, d = k_seqs[0].shape[1:]
    dv = v_seqs[0].shape[2]
    dtype = dtype or k_seqs[0].dtype
    k_cache = torch.full((num_pages, page, h, d), float("nan"), dtype=dtype)
    v_cache = torch.full((num_pages, page, h, dv), float("nan"), dtype=dtype)
    table = torch.zeros((len(lens), max(max(blocks), 1)), dtype=torch.int32)
    at = 0
    for b, (ks, vs) in enumerate(zip(k_seqs, v_seqs)):
        for j in range(blocks[b]):
            pg = perm[at].item()
            at += 1
            table[b, j] = pg
            chunk = slice(j * page, min((j + 1) * page, lens[b]))
            n = chunk.stop - chunk.start
            k_cache[pg, :n] = ks[chunk]
            v_cache[pg, :n] = vs[chunk]
    return k_cache, v_cache, table
