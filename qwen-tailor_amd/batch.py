"""Batched decode for B independent sequences at different positions: the call surface of qwen35/batch.py.

State lives in slot pools that the kernels update in place (qwen35/batch.py:1-18):
  ssm  : [S+1, 16, 128, 128] float32      slot s = one sequence
  conv : [(S+1)*2, 3, 6144]  bf16          double buffered: a step reads buffer pos&1 and writes the other one
  K, V : [S+1, 2, Lmax, 256] bf16          the attention kernel appends the new row of each sequence at its position
  slot S is the trash slot that padding rows point at.
All launches go to the current torch stream; in-place writes are ordered by stream order."""
from __future__ import annotations

import torch

from . import _lib as L
from .kernels import flat_conv_w
from .model import Cfg

BF16 = torch.bfloat16
HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224


def deltanet_b(proj, conv_pool, conv_w, A_log, dt_bias, ssm_pool, slots, pos, rows_per_wg: int = 0):
    """proj [B, 8224] bf16; slots / pos int32 [B] (pos = tokens already in the slot's state).  Returns y [B, 2048] bf16 and
    updates ssm_pool[slot] and the conv buffer (pos&1)^1 of the slot IN PLACE (qwen35/batch.py:128-135)."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    B = proj.shape[0]
    ssm_pool = L.dev(ssm_pool, torch.float32, "ssm_pool", (None, HV, DV, DK))
    n_slots = ssm_pool.shape[0]
    conv_pool = L.dev(conv_pool, BF16, "conv_pool", (n_slots * 2, 3, CD))
    slots, pos = L.i32(slots, "slots", B), L.i32(pos, "pos", B)
    w = flat_conv_w(conv_w)
    A, dtb = L.f32(A_log, "A_log", (HV,)), L.f32(dt_bias, "dt_bias", (HV,))
    y = torch.empty((B, HV * DV), dtype=BF16, device=proj.device)
    L.call("qt_gdn_decode_step", L.ptr(proj), L.ptr(conv_pool), L.ptr(w), L.ptr(A), L.ptr(dtb), L.ptr(ssm_pool), L.ptr(slots),
           L.ptr(pos), L.ptr(y), B, n_slots, rows_per_wg, L.stream())
    return y


_WORKSPACE = {}


def _workspace(dev, nbytes):
    """Split-K scratch of the attention kernel: one cached buffer per device, grown on demand (the C ABI never allocates)."""
    buf = _WORKSPACE.get(dev)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
        _WORKSPACE[dev] = buf
    return buf


def split_size(Lmax: int, B: int = 16) -> int:
    """Smallest number of pool keys a split-K workgroup takes.  The kernel spreads the batch's key tiles evenly over one
    workgroup per CU whatever the mix of lengths; this lower bound only matters for small batches of short sequences."""
    return 128


def attn_b(q, k, v, Kp, Vp, slots, pos, M=1, split=None):
    """q [R,H,D], k / v [R,KV,D] (normed + roped), pools [S+1,KV,Lmax,D]; R = B*M rows (row b*M+j = position pos[b]+j of slot
    slots[b]; slots / pos int32 [B]).  Returns o [R,H,D] bf16 and appends k / v at pos[b]+j (in place)
    (qwen35/batch.py:230-237)."""
    q = L.dev(q, BF16, "q", (None, 8, 256))
    R = q.shape[0]
    if M < 1 or M > 4 or R % M:
        raise ValueError(f"attn_b: M = {M} (1..4) must divide the number of rows ({R})")
    B = R // M
    k, v = L.dev(k, BF16, "k", (R, 2, 256)), L.dev(v, BF16, "v", (R, 2, 256))
    Kp = L.dev(Kp, BF16, "Kp", (None, 2, None, 256))
    Vp = L.dev(Vp, BF16, "Vp", tuple(Kp.shape))
    n_slots, Lmax = Kp.shape[0], Kp.shape[2]
    slots, pos = L.i32(slots, "slots", B), L.i32(pos, "pos", B)
    CH = split or split_size(Lmax, B)
    nbytes = L.lib().qt_gqa_attn_workspace_bytes(B, M, Lmax, CH)
    if nbytes < 0:
        raise ValueError("attn_b: bad split size")
    ws = _workspace(q.device, nbytes)
    o = torch.empty((R, 8, 256), dtype=BF16, device=q.device)
    L.call("qt_gqa_attn_decode", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(Kp), L.ptr(Vp), L.ptr(slots), L.ptr(pos), L.ptr(o), L.ptr(ws),
           ws.numel(), B, M, Lmax, n_slots, CH, L.stream())
    return o


def gnorm_rows(y, proj, gw, eps=1e-6):
    """Gated RMSNorm of the delta-rule output (qwen35/batch.py:338-343): y [B, 2048] bf16, proj [B, 8224] bf16 (its z slice
    is at 6144:8192), gw float32 [128].  Returns [B, 2048] bf16."""
    y = L.dev(y, BF16, "y", (None, HV * DV))
    B = y.shape[0]
    proj = L.dev(proj, BF16, "proj", (B, PW))
    gw = L.f32(gw, "gw", (DV,))
    out = torch.empty_like(y)
    L.call("qt_gated_rmsnorm", L.ptr(y), L.ptr(proj), L.ptr(gw), L.ptr(out), B, float(eps), L.stream())
    return out


class Pools:
    """Slot-major state pools of the batched decode step (qwen35/batch.py:405-462)."""

    def __init__(self, cfg: Cfg, slots: int, max_len: int, device="cuda"):
        self.cfg, self.S, self.Lmax = cfg, slots, max_len
        nl = sum(cfg.is_linear(i) for i in range(cfg.layers))
        na = cfg.layers - nl
        z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=device)
        self.conv = [z(((slots + 1) * 2, 3, CD), BF16) for _ in range(nl)]
        self.ssm = [z((slots + 1, HV, DV, DK), torch.float32) for _ in range(nl)]
        self.K = [z((slots + 1, cfg.n_kv, max_len, cfg.head_dim), BF16) for _ in range(na)]
        self.V = [z((slots + 1, cfg.n_kv, max_len, cfg.head_dim), BF16) for _ in range(na)]

    def nbytes(self):
        return sum(a.numel() * a.element_size() for g in (self.conv, self.ssm, self.K, self.V) for a in g)

    @staticmethod
    def slot_bytes(cfg: Cfg, max_len: int, double_conv=True):
        """Bytes one sequence occupies in the pools (qwen35/batch.py:420-426)."""
        nl = sum(cfg.is_linear(i) for i in range(cfg.layers))
        na = cfg.layers - nl
        return (nl * (HV * DV * DK * 4 + (2 if double_conv else 1) * 3 * CD * 2)
                + na * 2 * cfg.n_kv * max_len * cfg.head_dim * 2)

    def as_tree(self):
        return {"conv": self.conv, "ssm": self.ssm, "K": self.K, "V": self.V}

    def load(self, slot: int, state: dict, pos: int):
        """Copy a prefilled single-sequence state (kv [1,2,max_len,256] pairs, conv [1,3,6144], ssm [1,16,128,128], valid after
        `pos` tokens) into `slot`, in place (qwen35/batch.py:431-447)."""
        assert 0 <= slot < self.S and 0 < pos <= self.Lmax, (slot, pos)
        par = pos & 1
        for i, (c, s) in enumerate(zip(state["conv"], state["ssm"])):
            self.conv[i][slot * 2 + par].copy_(c.reshape(3, CD))
            self.ssm[i][slot].copy_(s.reshape(HV, DV, DK))
        for i, (K, V) in enumerate(state["kv"]):
            self.K[i][slot, :, :pos].copy_(K[0, :, :pos])
            self.V[i][slot, :, :pos].copy_(V[0, :, :pos])

    def read(self, slot: int, pos: int, max_len: int | None = None):
        """The slot's state as a single-sequence state dict of fresh tensors (qwen35/batch.py:449-462)."""
        ml = max_len or self.Lmax
        par = pos & 1
        st = {"kv": [], "conv": [c[slot * 2 + par][None].clone() for c in self.conv],
              "ssm": [s[slot][None].clone() for s in self.ssm]}
        for K, V in zip(self.K, self.V):
            def one(P):
                n = min(pos, ml)
                out = torch.zeros((1, P.shape[1], ml, P.shape[3]), dtype=P.dtype, device=P.device)
                out[0, :, :n].copy_(P[slot, :, :n])
                return out
            st["kv"].append((one(K), one(V)))
        return st
