"""Prefill glue of the GatedDeltaNet layer: conv + SiLU + q/k norm over S tokens and the gated RMSNorm
(qwen35/prefill.py:228-244)."""
from __future__ import annotations

import torch

from . import _lib as L
from .kernels import flat_conv_w

BF16 = torch.bfloat16
HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224


def conv_prep(proj, conv_state, conv_w):
    """proj [S,8224], conv_state [3,6144] -> q,k [S,16,128] (normalized, scaled), v [S,16,128]  (qwen35/prefill.py:228-238)."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    S = proj.shape[0]
    cs = L.dev(conv_state, BF16, "conv_state", (3, CD))
    w = flat_conv_w(conv_w)
    q, k, v = (torch.empty((S, HV, DK), dtype=BF16, device=proj.device) for _ in range(3))
    L.call("qt_gdn_conv_prep", L.ptr(proj), L.ptr(cs), L.ptr(w), L.ptr(q), L.ptr(k), L.ptr(v), S, L.stream())
    return q, k, v


def gated_norm(y, proj, gw):
    """Gated RMSNorm for S tokens (qwen35/prefill.py:241-244): y [S,16,128] or [S,2048] bf16 -> [S,2048] bf16."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    S = proj.shape[0]
    y = L.dev(y, BF16, "y").reshape(S, HV * DV)
    gw = L.f32(gw, "gw", (DV,))
    out = torch.empty((S, HV * DV), dtype=BF16, device=proj.device)
    L.call("qt_gated_rmsnorm", L.ptr(y), L.ptr(proj), L.ptr(gw), L.ptr(out), S, 1e-6, L.stream())
    return out
