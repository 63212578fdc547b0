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


_WS_MIN = 32 << 20       # first allocation of the attention scratch: enough for 256 sequences x 4 rows, so that growth is rare


def _workspace(dev, nbytes):
    """Split-K scratch of the attention kernel, cached per (device, stream) (see _lib.workspace).  Callers that manage memory
    themselves pass `workspace=` to attn_b instead."""
    return L.workspace("attn_b", dev, nbytes, _WS_MIN)


def deltanet_b_gnorm(proj, conv_pool, conv_w, A_log, dt_bias, ssm_pool, slots, pos, gw, eps=1e-6):
    """deltanet_b followed by gnorm_rows (qwen35/batch.py:128-135, 338-343; the two calls of the reference's decode step,
    batch.py:497-499) in one launch.  Returns the gated-norm output [B, 2048] bf16 (the same bits as the two calls); pools are
    updated in place as by deltanet_b."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    B = proj.shape[0]
    ssm_pool = L.dev(ssm_pool, torch.float32, "ssm_pool", (None, HV, DV, DK))
    n_slots = ssm_pool.shape[0]
    conv_pool = L.dev(conv_pool, BF16, "conv_pool", (n_slots * 2, 3, CD))
    slots, pos = L.i32(slots, "slots", B), L.i32(pos, "pos", B)
    w = flat_conv_w(conv_w)
    A, dtb, gw = L.f32(A_log, "A_log", (HV,)), L.f32(dt_bias, "dt_bias", (HV,)), L.f32(gw, "gw", (DV,))
    out = torch.empty((B, HV * DV), dtype=BF16, device=proj.device)
    L.call("qt_gdn_decode_step_gnorm", L.ptr(proj), L.ptr(conv_pool), L.ptr(w), L.ptr(A), L.ptr(dtb), L.ptr(ssm_pool), L.ptr(slots),
           L.ptr(pos), L.ptr(gw), float(eps), L.ptr(out), B, n_slots, L.stream())
    return out


def split_size(Lmax: int, B: int = 16) -> int:
    """Smallest number of pool keys a split-K workgroup takes.  The kernel spreads the batch's key tiles evenly over one
    workgroup per CU whatever the mix of lengths; this lower bound only matters for small batches of short sequences."""
    return 128


def attn_b(q, k, v, Kp, Vp, slots, pos, M=1, split=None, workspace=None):
    """q [R,H,D], k / v [R,KV,D] (normed + roped), pools [S+1,KV,Lmax,D]; R = B*M rows (row b*M+j = position pos[b]+j of slot
    slots[b]; slots / pos int32 [B]).  Returns o [R,H,D] bf16 and appends k / v at pos[b]+j (in place)
    (qwen35/batch.py:230-237).  M up to 16 (the limit of batch_spec.deltanet_bm); more than four tokens per sequence run as
    passes of four, each reading the pool once.  workspace: optional uint8 device tensor of at least qt_gqa_attn_workspace_bytes(B, M, Lmax, split)
    bytes for the split-K partial results (default: a buffer cached per device and stream)."""
    q = L.dev(q, BF16, "q", (None, 8, 256))
    R = q.shape[0]
    if M < 1 or M > 16 or R % M:
        raise ValueError(f"attn_b: M = {M} (1..16, as deltanet_bm) must divide the number of rows ({R})")
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
    if workspace is None:
        ws = _workspace(q.device, nbytes)
    else:
        ws = L.dev(workspace, torch.uint8, "workspace")
        if ws.numel() < nbytes:
            raise ValueError(f"attn_b: workspace of {ws.numel()} bytes, {nbytes} needed")
    o = torch.empty((R, 8, 256), dtype=BF16, device=q.device)
    L.call("qt_gqa_attn_decode", L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(Kp), L.ptr(Vp), L.ptr(slots), L.ptr(pos), L.ptr(o), L.ptr(ws),
           ws.numel(), B, M, Lmax, n_slots, CH, L.stream())
    return o


def attn_layer_b(qkv, q_norm, k_norm, Kp, Vp, slots, pos, M=1, eps=1e-6, split=None, workspace=None):
    """The attention half of a full-attention layer at a decode / verify step (qwen35/batch.py:505-513), between the qkv and o
    projections: q / k RMSNorm and rotary embedding, attn_b, and o * sigmoid(gate), in two launches per pass of four tokens
    (attention.qkv_prep + attn_b + attention.out_gate are four), with the same bits.  qkv [B*M,5120] bf16 = [(q_h | gate_h) x 8 |
    k x 2 | v x 2]; q_norm, k_norm [256] bf16; pools, slots, pos, M as for attn_b (the new K / V rows are appended in place).
    Returns [B*M,2048] bf16.  The first call on a device (and the first one with a longer pool) builds the rotary table: make
    it outside HIP graph capture."""
    qkv = L.dev(qkv, BF16, "qkv", (None, 5120))
    R = qkv.shape[0]
    if M < 1 or M > 16 or R % M:
        raise ValueError(f"attn_layer_b: M = {M} (1..16) must divide the number of rows ({R})")
    B = R // M
    qn, kn = L.dev(q_norm, BF16, "q_norm", (256,)), L.dev(k_norm, BF16, "k_norm", (256,))
    Kp = L.dev(Kp, BF16, "Kp", (None, 2, None, 256))
    Vp = L.dev(Vp, BF16, "Vp", tuple(Kp.shape))
    n_slots, Lmax = Kp.shape[0], Kp.shape[2]
    slots, pos = L.i32(slots, "slots", B), L.i32(pos, "pos", B)
    CH = split or split_size(Lmax, B)
    nbytes = L.lib().qt_gqa_attn_workspace_bytes(B, M, Lmax, CH)
    if nbytes < 0:
        raise ValueError("attn_layer_b: bad split size")
    if workspace is None:
        ws = _workspace(qkv.device, nbytes)
    else:
        ws = L.dev(workspace, torch.uint8, "workspace")
        if ws.numel() < nbytes:
            raise ValueError(f"attn_layer_b: workspace of {ws.numel()} bytes, {nbytes} needed")
    table, n_pos = L.rope_table(qkv.device, Lmax)
    out = torch.empty((R, 2048), dtype=BF16, device=qkv.device)
    L.call("qt_gqa_attn_layer_decode", L.ptr(qkv), L.ptr(qn), L.ptr(kn), L.ptr(table), n_pos, L.ptr(Kp), L.ptr(Vp), L.ptr(slots),
           L.ptr(pos), L.ptr(out), L.ptr(ws), ws.numel(), B, M, Lmax, n_slots, CH, float(eps), L.stream())
    return out


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


def rms_rows(x, nw, eps=1e-6, T=128, f32=False):
    """qwen35/batch.py:295-301; see kernels.rms_rows."""
    from .kernels import rms_rows as _rms_rows
    return _rms_rows(x, nw, eps, T, f32)


def blit(dst, src, n, d0, s0, ny=1, dstride=0, sstride=0):
    """dst.flat[d0 + y*dstride + i] = src.flat[s0 + y*sstride + i] for i < n, y < ny, in place (qwen35/batch.py:365-372).
    dst and src are contiguous device tensors of the same dtype (bf16 or float32); returns dst."""
    if dst.dtype != src.dtype or dst.dtype not in (BF16, torch.float32):
        raise TypeError(f"blit: bf16 or float32 tensors of one dtype expected, got {dst.dtype} and {src.dtype}")
    dst, src = L.dev(dst, dst.dtype, "dst"), L.dev(src, src.dtype, "src")
    n, d0, s0, ny, dstride, sstride = (int(x) for x in (n, d0, s0, ny, dstride, sstride))
    if n < 0 or ny < 0 or min(d0, s0, dstride, sstride) < 0:
        raise ValueError("blit: negative size, offset or stride")
    if n and ny and (d0 + (ny - 1) * dstride + n > dst.numel() or s0 + (ny - 1) * sstride + n > src.numel()):
        raise ValueError("blit: the copy leaves the source or the destination")
    L.call("qt_blit", L.ptr(dst), L.ptr(src), dst.element_size(), n, d0, s0, ny, dstride, sstride, L.stream())
    return dst


def blit_batch(jobs):
    """Several blits in one launch: jobs = [(dst, src, n, d0, s0, ny, dstride, sstride), ...] with the arguments of blit.
    Every copy must be 16-byte granular (a ValueError says which one is not)."""
    import ctypes
    k = len(jobs)
    if k == 0:
        return
    dsts, srcs, meta = (ctypes.c_void_p * k)(), (ctypes.c_void_p * k)(), (ctypes.c_long * (7 * k))()
    for i, (dst, src, n, d0, s0, ny, dstride, sstride) in enumerate(jobs):
        if dst.dtype != src.dtype or dst.dtype not in (BF16, torch.float32):
            raise TypeError(f"blit_batch: job {i}: bf16 or float32 tensors of one dtype expected")
        L.dev(dst, dst.dtype, "dst"), L.dev(src, src.dtype, "src")
        n, d0, s0, ny, dstride, sstride = (int(x) for x in (n, d0, s0, ny, dstride, sstride))
        if n < 0 or ny < 0 or min(d0, s0, dstride, sstride) < 0:
            raise ValueError(f"blit_batch: job {i}: negative size, offset or stride")
        if n and ny and (d0 + (ny - 1) * dstride + n > dst.numel() or s0 + (ny - 1) * sstride + n > src.numel()):
            raise ValueError(f"blit_batch: job {i}: the copy leaves the source or the destination")
        dsts[i], srcs[i] = dst.data_ptr(), src.data_ptr()
        meta[7 * i:7 * i + 7] = [dst.element_size(), n, d0, s0, ny, dstride, sstride]
    rc = L.lib().qt_blit_batch(dsts, srcs, meta, k, L.stream())
    if rc == -2:
        raise ValueError("blit_batch: every copy must be 16-byte granular (base pointers, sizes, offsets, strides)")
    if rc:
        raise RuntimeError(f"qt_blit_batch failed: {L.ERRORS.get(rc, rc)}")


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
        `pos` tokens) into `slot`, in place, with the strided copy kernel (qwen35/batch.py:431-447)."""
        assert 0 <= slot < self.S and 0 < pos <= self.Lmax, (slot, pos)
        par = pos & 1
        jobs = []
        for i, (c, s) in enumerate(zip(state["conv"], state["ssm"])):
            jobs.append((self.conv[i], c, CD * 3, (slot * 2 + par) * 3 * CD, 0, 1, 0, 0))
            jobs.append((self.ssm[i], s, HV * DV * DK, slot * HV * DV * DK, 0, 1, 0, 0))
        nkv, D = self.cfg.n_kv, self.cfg.head_dim
        for i, (K, V) in enumerate(state["kv"]):
            smax = K.shape[2]
            for pool, src in ((self.K[i], K), (self.V[i], V)):
                jobs.append((pool, src, pos * D, slot * nkv * self.Lmax * D, 0, nkv, self.Lmax * D, smax * D))
        blit_batch(jobs)                                         # one launch for the whole sequence (the reference issues 48 blits)

    def read(self, slot: int, pos: int, max_len: int | None = None):
        """The slot's state as a single-sequence state dict of fresh tensors (qwen35/batch.py:449-462): the inverse of load,
        one launch of the strided copy kernel; K / V rows from `pos` on are zero."""
        ml = max_len or self.Lmax
        par = pos & 1
        nkv, D = self.cfg.n_kv, self.cfg.head_dim
        n = min(pos, ml)
        st = {"kv": [], "conv": [torch.empty((1, 3, CD), dtype=BF16, device=c.device) for c in self.conv],
              "ssm": [torch.empty((1, HV, DV, DK), dtype=torch.float32, device=s.device) for s in self.ssm]}
        jobs = []
        for i in range(len(self.conv)):
            jobs.append((st["conv"][i], self.conv[i], 3 * CD, 0, (slot * 2 + par) * 3 * CD, 1, 0, 0))
            jobs.append((st["ssm"][i], self.ssm[i], HV * DV * DK, 0, slot * HV * DV * DK, 1, 0, 0))
        for K, V in zip(self.K, self.V):
            pair = []
            for P in (K, V):
                out = torch.zeros((1, nkv, ml, D), dtype=P.dtype, device=P.device)
                if n:
                    jobs.append((out, P, n * D, 0, slot * nkv * self.Lmax * D, nkv, ml * D, self.Lmax * D))
                pair.append(out)
            st["kv"].append(tuple(pair))
        blit_batch(jobs)
        return st
