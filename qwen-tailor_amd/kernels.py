"""kernels.deltanet: the fused decode / verify GatedDeltaNet step for one sequence (qwen35/kernels.py:555-567)."""
from __future__ import annotations

import torch

from . import _lib as L

BF16 = torch.bfloat16
HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224


def flat_conv_w(conv_w):
    """conv_w arrives as [6144, 4, 1] (or [6144, 4]); tap j of channel ch sits at ch*4 + j (qwen35/model.py:86)."""
    w = L.dev(conv_w, BF16, "conv_w")
    if w.numel() != CD * 4:
        raise ValueError(f"conv_w: expected {CD * 4} elements, got {w.numel()}")
    return w


def deltanet(proj, conv_snap, conv_w, A_log, dt_bias, ssm_snap, sel, rows_per_wg: int = 0):
    """proj [M, 8224] bf16 (qkv 6144 | z 2048 | b 16 | a 16 per token).
    conv_snap [S,3,6144] / ssm_snap [S,16,128,128]: state snapshots; the step starts from snapshot sel[0].
    Returns y [M,2048], conv snapshots [M,3,6144] (after each token), ssm snapshots [M,16,128,128]."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    M = proj.shape[0]
    conv_snap = L.dev(conv_snap, BF16, "conv_snap", (None, 3, CD))
    ssm_snap = L.dev(ssm_snap, torch.float32, "ssm_snap", (None, HV, DV, DK))
    S = ssm_snap.shape[0]
    if conv_snap.shape[0] != S:
        raise ValueError("conv_snap and ssm_snap must hold the same number of snapshots")
    sel = L.i32(sel, "sel", 1)
    w = flat_conv_w(conv_w)
    A, dtb = L.f32(A_log, "A_log", (HV,)), L.f32(dt_bias, "dt_bias", (HV,))
    y = torch.empty((M, HV * DV), dtype=BF16, device=proj.device)
    cs = torch.empty((M, 3, CD), dtype=BF16, device=proj.device)
    st = torch.empty((M, HV, DV, DK), dtype=torch.float32, device=proj.device)
    L.call("qt_gdn_deltanet", L.ptr(proj), L.ptr(conv_snap), L.ptr(w), L.ptr(A), L.ptr(dtb), L.ptr(ssm_snap), L.ptr(sel),
           L.ptr(y), L.ptr(cs), L.ptr(st), M, S, rows_per_wg, L.stream())
    return y, cs, st
