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
    # launches that would leave half of the CUs idle are split along the keys; their parts meet in a workspace
    nws = L.lib().qt_gqa_prefill_workspace_bytes_for(S, Lk, Lk - S)
    ws = L.workspace("prefill_attention", q.device, nws) if nws > 0 else None      # cached per (device, stream)
    L.call("qt_gqa_prefill_causal", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(out), L.ptr(ws), max(nws, 0),
           S, Lk, Lk - S, S * 256, k.stride(1), L.stream())
    return out


QKV_W = 8 * 512 + 2 * 2 * 256


def qkv_prep(qkv, q_norm, k_norm, pos, M=1, eps=1e-6, max_pos=None):
    """The steps between the qkv projection and the attention kernel of a full-attention layer (qwen35/batch.py:505-512,
    qwen35/model.py:154-164): split the 5120-wide rows into q / gate / k / v, RMS-normalise q and k per head (weights [256]
    bf16), rotate their first 64 features to the row's position.  qkv [R,5120] bf16, pos int32 [R / M] (row b*M + j sits at
    pos[b] + j).  Returns q [R,8,256], k [R,2,256], v [R,2,256] bf16; the gate stays in qkv (out_gate reads it there).
    max_pos: a bound of the positions that the caller knows on the host (a prefill knows its key count): the rotary (cos,
    sin) pairs then come from the device's table of positions 0 .. max_pos instead of being evaluated per row (same bits;
    a row beyond the bound still evaluates its own)."""
    qkv = L.dev(qkv, BF16, "qkv", (None, QKV_W))
    R = qkv.shape[0]
    if M < 1 or R % M:
        raise ValueError(f"qkv_prep: M = {M} must divide the number of rows ({R})")
    pos = L.i32(pos, "pos", R // M)
    qn, kn = L.dev(q_norm, BF16, "q_norm", (256,)), L.dev(k_norm, BF16, "k_norm", (256,))
    q = torch.empty((R, 8, 256), dtype=BF16, device=qkv.device)
    k, v = (torch.empty((R, 2, 256), dtype=BF16, device=qkv.device) for _ in range(2))
    if max_pos is None:
        L.call("qt_attn_qkv_prep", L.ptr(qkv), L.ptr(qn), L.ptr(kn), L.ptr(pos), L.ptr(q), L.ptr(k), L.ptr(v), R, M, float(eps), L.stream())
    else:
        table, n_pos = L.rope_table(qkv.device, int(max_pos) + 1)
        L.call("qt_attn_qkv_prep_table", L.ptr(qkv), L.ptr(qn), L.ptr(kn), L.ptr(pos), L.ptr(table), n_pos, L.ptr(q), L.ptr(k), L.ptr(v),
               R, M, float(eps), L.stream())
    return q, k, v


def out_gate(o, qkv):
    """o * sigmoid(gate) (qwen35/batch.py:513): o [R,8,256] bf16, qkv [R,5120] bf16 -> [R,2048] bf16"""
    qkv = L.dev(qkv, BF16, "qkv", (None, QKV_W))
    R = qkv.shape[0]
    o = L.dev(o, BF16, "o", (R, 8, 256))
    out = torch.empty((R, 2048), dtype=BF16, device=qkv.device)
    L.call("qt_attn_out_gate", L.ptr(o), L.ptr(qkv), L.ptr(out), R, L.stream())
    return out
