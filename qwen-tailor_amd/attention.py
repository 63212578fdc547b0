"""Causal prefill attention of the full-attention layers: stands where the reference calls
mx.fast.scaled_dot_product_attention(q, K[:, :, :kv_len], V[:, :, :kv_len], scale=D**-0.5, mask="causal")
(qwen35/model.py:160-167, qwen35/prefill.py:468).  8 query heads on 2 KV heads, head dim 256."""
from __future__ import annotations

import torch

from . import _lib as L

BF16 = torch.bfloat16


def scaled_dot_product_attention(q, k, v, *, scale: float, mask="causal"):
    """q [1, 8, S, 256], k / v [1, 2, L, 256] bf16 (k, v may be length-slices of a longer cache).  mask = "causal": query i
    sits at position L - S + i and sees keys 0 .. L - S + i.  Returns [1, 8, S, 256] bf16."""
    if mask != "causal":
        raise ValueError("only mask='causal' is built (decode / verify rows go through batch.attn_b)")
    if abs(scale - 256 ** -0.5) > 1e-9:
        raise ValueError("only scale = 256**-0.5 is built")
    if q.dim() != 4 or q.shape[0] != 1 or q.shape[1] != 8 or q.shape[3] != 256 or q.dtype != BF16 or not q.is_cuda:
        raise ValueError(f"q: expected [1, 8, S, 256] bf16 on the GPU, got {tuple(q.shape)} {q.dtype}")
    S = q.shape[2]
    for t, name in ((k, "k"), (v, "v")):
        if t.dim() != 4 or t.shape[0] != 1 or t.shape[1] != 2 or t.shape[3] != 256 or t.dtype != BF16 or not t.is_cuda:
            raise ValueError(f"{name}: expected [1, 2, L, 256] bf16 on the GPU")
        if t.stride(3) != 1 or t.stride(2) != 256:
            raise ValueError(f"{name}: rows must be contiguous")
    if k.shape != v.shape or k.stride(1) != v.stride(1):
        raise ValueError("k and v must have the same shape and head stride")
    Lk = k.shape[2]
    if Lk < S:
        raise ValueError("fewer keys than queries")
    q = q.contiguous()
    out = torch.empty_like(q)
    L.call("qt_gqa_prefill_causal", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(out), None, 0, S, Lk, Lk - S, S * 256, k.stride(1),
           L.stream())
    return out
