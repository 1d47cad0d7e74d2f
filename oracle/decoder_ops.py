"""Oracle for the decoder-layer helpers (test infrastructure): KV-cache fill, RMSNorm and
rotary embedding, each a restatement of the ground truth in the reference's own test:

* ``fill_kv_cache``  python/dlBLAS/tests/kernels/test_fill_kv_cache.py:109-137 (python loop
  copying each sequence's new tokens page by page, starting at ``history % block_size``);
* ``rms_norm``       python/dlBLAS/tests/kernels/test_rms_norm.py:25-30
  (``weight * (x.float() * rsqrt(mean(x^2) + eps)).to(dtype)``); with a residual the input is
  ``x + residual`` first (python/dlBLAS/dlblas/kernels/rms_norm.py:57-60);
* ``apply_rotary_pos_emb``  python/dlBLAS/tests/kernels/test_apply_rotary.py:7-11,66-69
  (``x * cos + rotate_half(x) * sin``).
"""
from __future__ import annotations

import torch


def fill_kv_cache(k_states, v_states, k_caches, v_caches, seq_lens, history_lens, block_offsets):
    block_size = k_caches.shape[1]
    k_caches, v_caches = k_caches.clone(), v_caches.clone()
    ks_split = k_states.split(list(seq_lens))
    vs_split = v_states.split(list(seq_lens))
    for b, (ks, vs) in enumerate(zip(ks_split, vs_split)):
        for i in range(ks.shape[0]):                      # one token at a time: no page logic to get wrong
            pos = history_lens[b] + i
            page = int(block_offsets[b][pos // block_size])
            k_caches[page, pos % block_size] = ks[i]
            v_caches[page, pos % block_size] = vs[i]
    return k_caches, v_caches


def rms_norm(x, weight, eps=1e-6, residual=None):
    dt = x.dtype
    if residual is not None:
        x = (x.float() + residual.float()).to(dt)
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    out = weight * (xf * torch.rsqrt(var + eps)).to(dt)
    return out if residual is None else (out, x)


def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin):
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin
