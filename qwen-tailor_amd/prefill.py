"""Prefill glue of the GatedDeltaNet layer: conv + SiLU + q/k norm over S tokens and the gated RMSNorm
(qwen35/prefill.py:228-244)."""
from __future__ import annotations

import torch

from . import _lib as L
from .kernels import flat_conv_w

BF16 = torch.bfloat16
HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224


import os

from . import gated_delta, gdn_nax

# GatedDeltaNet prefill recurrence: "nax" = chunked two-phase MFMA kernels (gdn_nax.py), "ref" = the sequential kernel
# (gated_delta.py); same switch as the reference's QWEN35_GDN (qwen35/prefill.py:15-16)
GDN_IMPL = os.environ.get("QWEN35_GDN", "nax")


def gdn_core(proj, conv_state, ssm_state, conv_w, A_log, dt_bias, gnorm, want_qkv=False):
    """The GatedDeltaNet layer core over S tokens, between the in_proj and out_proj GEMMs of prefill._linear_attn
    (qwen35/prefill.py:247-265): proj [S,8224] bf16, conv_state [1,3,6144] bf16, ssm_state [1,16,128,128] f32 ->
    (gated-norm output [S,2048] bf16, new conv state [1,3,6144], new ssm state [1,16,128,128])."""
    S = proj.shape[0]
    cs = conv_state.reshape(3, CD)
    if GDN_IMPL == "nax":
        new_conv = torch.empty((1, 3, CD), dtype=BF16, device=proj.device)
        _, _, _, ops, U, gC = gdn_nax._phase_a(proj, cs, conv_w, A_log, dt_bias, want_qkv=want_qkv, conv_out=new_conv[0])
        normed, new_ssm = gdn_nax.phase_b_norm(proj, ops, U, gC, ssm_state, gnorm)
    else:
        q, k, v = conv_prep(proj, cs, conv_w)
        out, new_ssm = gated_delta.gated_delta_update(q[None], k[None], v[None], proj[:, 8208:][None], proj[:, 8192:8208][None],
                                                      A_log, dt_bias, ssm_state.reshape(1, HV, DV, DK))
        normed = gated_norm(out.reshape(S, HV * DV), proj, gnorm)
        tail = proj[:, :CD]
        new_conv = (tail[S - 3:] if S >= 3 else torch.cat([cs, tail], dim=0)[-3:])[None].contiguous()   # prefill.py:262-263
    return normed, new_conv, new_ssm.reshape(1, HV, DV, DK)


def conv_prep(proj, conv_state, conv_w):
    """proj [S,8224], conv_state [3,6144] -> q,k [S,16,128] (normalized, scaled), v [S,16,128]  (qwen35/prefill.py:228-238)."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    S = proj.shape[0]
    cs = L.dev(conv_state, BF16, "conv_state", (3, CD))
    w = flat_conv_w(conv_w)
    q, k, v = (torch.empty((S, HV, DK), dtype=BF16, device=proj.device) for _ in range(3))
    L.call("qt_gdn_conv_prep", L.ptr(proj), L.ptr(cs), L.ptr(w), L.ptr(L.silu_table(proj.device)), L.ptr(q), L.ptr(k), L.ptr(v), S,
           L.stream())
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
