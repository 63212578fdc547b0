"""kernels.deltanet: the fused decode / verify GatedDeltaNet step for one sequence (qwen35/kernels.py:555-567);
kernels.fused_gemv: the projections either side of the core (qwen35/kernels.py:291-319)."""
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


def rms_rows(x, nw, eps=1e-6, T=None, f32=False):
    """The rms prologue of fused_gemv as its own kernel (qwen35/batch.py:295-301): x [M, K] bf16, nw [K] bf16 ->
    BF(nw * (x * rsqrt(mean(x^2) + eps))) [M, K].  T (the reference's threadgroup size) does not change the result and is
    ignored.  f32=True returns the same bf16 values widened to float32, as the reference does."""
    x = L.dev(x, BF16, "x", (None, None))
    M, K = x.shape
    nw = L.dev(nw, BF16, "nw", (K,))
    y = torch.empty_like(x)
    L.call("qt_rms_rows", L.ptr(x), L.ptr(nw), L.ptr(y), M, K, float(eps), L.stream())
    return y.float() if f32 else y


def fused_gemv(W, x, *, nw=None, eps=1e-6, res=None, swiglu=False, gnorm=None, T=None, R=None, mtmax=None, wf=False):
    """y = W @ f(x) (qwen35/kernels.py:291-319).  W [N, K] bf16; x [..., K] bf16, or float32 holding bf16 values (what
    rms_rows(f32=True) returns).  nw: rms prologue weight [K]; gnorm = (proj [M, 8224], gw [128]): gated-norm prologue
    (K = 2048); res [..., N]: residual added after rounding the product to bf16; swiglu: rows of W interleave gate and up,
    the result is [..., N/2].  T, R, mtmax, wf are the reference's tilings: they never change its arithmetic and are ignored.
    Weights in the reference's lossless 12-bit form are not taken: pass the plain bf16 matrix."""
    if isinstance(W, (tuple, list)):
        raise TypeError("W: compressed weight pairs are not supported, pass the plain bf16 [N, K] matrix")
    W = L.dev(W, BF16, "W", (None, None))
    N, K = W.shape
    if not isinstance(x, torch.Tensor) or not x.is_cuda:
        raise TypeError("x: expected a tensor on the GPU")
    if x.shape[-1] != K:
        raise ValueError(f"x: last dimension must be {K}, got {tuple(x.shape)}")
    lead = tuple(x.shape[:-1])
    if x.dtype == torch.float32:
        if nw is not None or gnorm is not None:
            raise ValueError("float32 x carries already normalised values: no prologue may follow")
        x = x.to(BF16)                                           # exact: the values are bf16 values
    x = L.dev(x.reshape(-1, K), BF16, "x", (None, K))
    M = x.shape[0]
    if nw is not None and gnorm is not None:
        raise ValueError("nw and gnorm are exclusive")
    if swiglu and res is not None:
        raise ValueError("swiglu and res are exclusive")
    if nw is not None:
        x = rms_rows(x, nw, eps)
    if gnorm is not None:
        from .batch import gnorm_rows
        x = gnorm_rows(x, gnorm[0].reshape(M, PW), gnorm[1], eps)
    epi = 2 if swiglu else (1 if res is not None else 0)
    n_out = N // 2 if swiglu else N
    if res is not None:
        res = L.dev(res.reshape(-1, N), BF16, "res", (M, N))
    y = torch.empty((M, n_out), dtype=BF16, device=x.device)
    L.call("qt_fused_gemv", L.ptr(W), L.ptr(x), L.ptr(res), L.ptr(y), M, N, K, epi, L.stream())
    return y.reshape(*lead, n_out)
