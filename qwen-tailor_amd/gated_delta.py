"""The gated delta rule recurrence and the q/k normalisation: the call surface of qwen35/gated_delta.py on torch tensors."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib as L

BF16 = torch.bfloat16


def _gates(A_log, a, b, dt_bias, want_g=True, want_lg=False, want_beta=True):
    """a, b: [..., Hv] bf16 views whose last dim is contiguous and whose leading dims collapse to one row stride."""
    hv = a.shape[-1]
    rows = a.numel() // hv

    def rows_view(t, name):
        if t.dtype != BF16 or not t.is_cuda:
            raise TypeError(f"{name}: expected a bf16 tensor on the GPU")
        t2 = t.reshape(rows, hv) if t.is_contiguous() else t
        if t2.dim() != 2:
            t2 = t.contiguous().reshape(rows, hv)
        if t2.stride(1) != 1:
            t2 = t2.contiguous()
        return t2

    a2 = rows_view(a, "a")
    b2 = rows_view(b, "b") if b is not None else None
    A = L.f32(A_log, "A_log", (hv,))
    dtb = L.f32(dt_bias, "dt_bias", (hv,))
    g = torch.empty(a.shape, dtype=torch.float32, device=a.device) if want_g else None
    lg = torch.empty(a.shape, dtype=torch.float32, device=a.device) if want_lg else None
    beta = torch.empty(a.shape, dtype=BF16, device=a.device) if (want_beta and b is not None) else None
    L.call("qt_gdn_gates", L.ptr(a2), L.ptr(b2), a2.stride(0), b2.stride(0) if b2 is not None else 0, L.ptr(A), L.ptr(dtb),
           L.ptr(g), L.ptr(lg), L.ptr(beta), rows, hv, L.stream())
    return g, lg, beta


def compute_g(A_log, a, dt_bias):
    """g = exp(-exp(A_log) * softplus(a + dt_bias)), float32 (qwen35/gated_delta.py:16-18)."""
    return _gates(A_log, a, None, dt_bias, want_beta=False)[0]


def normalize_qk(q, k, *, inv_scale: float, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """L2-normalise q / k over the last dim (128) and fold the 128^-0.5 read-out scale into q
    (qwen35/gated_delta.py:21-30).  Only inv_scale = 128^-0.5, eps = 1e-6 is built."""
    if q.shape[-1] != 128 or k.shape[-1] != 128 or abs(inv_scale - 128 ** -0.5) > 1e-9 or abs(eps - 1e-6) > 1e-12:
        raise ValueError("normalize_qk: only head dim 128, inv_scale = 128**-0.5, eps = 1e-6 is supported")
    if q.shape != k.shape:
        raise ValueError("normalize_qk: q and k must have the same shape")
    q, k = L.dev(q, BF16, "q"), L.dev(k, BF16, "k")
    qo, ko = torch.empty_like(q), torch.empty_like(k)
    L.call("qt_normalize_qk", L.ptr(q), L.ptr(k), L.ptr(qo), L.ptr(ko), q.numel() // 128, 128, L.stream())
    return qo, ko


def gated_delta_update(q, k, v, a, b, A_log, dt_bias, state: Optional[torch.Tensor] = None):
    """Gated delta rule over T tokens (qwen35/gated_delta.py:143-174).

    q, k: [B, T, Hk, Dk] bf16 (already through normalize_qk); v: [B, T, Hv, Dv] bf16; a, b: [B, T, Hv] bf16;
    state: [B, Hv, Dv, Dk] float32 (zeros if None).  Returns (y [B, T, Hv, Dv] bf16, new state float32)."""
    B, T, Hk, Dk = k.shape
    Hv, Dv = v.shape[2:]
    if state is None:
        state = torch.zeros((B, Hv, Dv, Dk), dtype=torch.float32, device=q.device)
    if Dk != 128 or Dv % 8 or state.dtype != torch.float32:
        raise ValueError(f"only the scalar-gate, Dk=128, fp32-state case is supported (Dk={Dk}, Dv={Dv}, state {state.dtype})")
    if Hv % Hk:
        raise ValueError(f"unsupported head layout (Hk={Hk}, Hv={Hv}, Dv={Dv})")
    q, k, v = L.dev(q, BF16, "q", (B, T, Hk, Dk)), L.dev(k, BF16, "k"), L.dev(v, BF16, "v", (B, T, Hv, Dv))
    state = L.dev(state, torch.float32, "state", (B, Hv, Dv, Dk))
    g, _, beta = _gates(A_log, a, b, dt_bias)
    y = torch.empty((B, T, Hv, Dv), dtype=BF16, device=q.device)
    out = torch.empty_like(state)
    L.call("qt_gdn_recurrent", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(g), L.ptr(beta), L.ptr(state), L.ptr(out), L.ptr(y),
           B, T, Hk, Hv, Dk, Dv, L.stream())
    return y, out
