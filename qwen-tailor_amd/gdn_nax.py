"""Two-phase chunked gated-delta-rule for prefill: the call surface of qwen35/gdn_nax.py (prep_a, phase_b, gdn_chunked).

Chunk size is 64 (the reference's is 16; the chunked form is an identity for every chunk size).  The three buffers that
travel from phase A to phase B keep the reference's argument slots (Tbuf, Abuf, gv) but hold this implementation's own
records: the packed half-precision MFMA operands, the U tiles (half precision), and the per-token / per-chunk decay factors."""
from __future__ import annotations

import torch

from . import _lib as L
from .kernels import flat_conv_w

BF16 = torch.bfloat16
HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224
CHUNK = 64

# precision flags of the reference (qwen35/gdn_nax.py:363-366) are accepted and ignored: the operands are always fp16
FLAGS = ("RNE", "SPLIT_P1", "SPLIT_P2", "SPLIT_D", "SPLIT_Y", "SPLIT_DP", "PF")
DEFAULT_FLAGS = frozenset()
TG = 64


def _alloc_records(S, dev):
    lib = L.lib()
    ops = torch.empty(lib.qt_gdn_chunk_ops_bytes(S) // 2, dtype=torch.float16, device=dev)
    U = torch.empty(lib.qt_gdn_chunk_u_bytes(S) // 2, dtype=torch.float16, device=dev)
    gC = torch.empty(lib.qt_gdn_chunk_gc_bytes(S) // 4, dtype=torch.float32, device=dev)
    return ops, U, gC


def _phase_a(proj, conv_state, conv_w, A_log, dt_bias, qkv=None, want_qkv=True, conv_out=None):
    """Phase A.  With q, k, v given: the kernel that consumes them.  Otherwise one kernel that convolves and normalizes the
    projection rows itself (returning q, k, v only if want_qkv) and, if conv_out [3,6144] is given, writes the new conv
    window there.  Returns (q, k, v, ops, U, gC)."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    S = proj.shape[0]
    A, dtb = L.f32(A_log, "A_log", (HV,)), L.f32(dt_bias, "dt_bias", (HV,))
    ops, U, gC = _alloc_records(S, proj.device)
    if qkv is not None:
        q, k, v = (L.dev(t, BF16, name, (S, HV, DK)) for t, name in zip(qkv, "qkv"))
        L.call("qt_gdn_phase_a", L.ptr(proj), L.ptr(q), L.ptr(k), L.ptr(v), L.ptr(A), L.ptr(dtb), L.ptr(ops), L.ptr(U), L.ptr(gC), S,
               L.stream())
        return q, k, v, ops, U, gC
    cs = L.dev(conv_state, BF16, "conv_state", (3, CD))
    w = flat_conv_w(conv_w)
    q = k = v = None
    if want_qkv:
        q, k, v = (torch.empty((S, HV, DK), dtype=BF16, device=proj.device) for _ in range(3))
    if conv_out is not None:
        conv_out = L.dev(conv_out, BF16, "conv_out", (3, CD))
    L.call("qt_gdn_phase_a_conv", L.ptr(proj), L.ptr(cs), L.ptr(w), L.ptr(L.silu_table(proj.device)), L.ptr(A), L.ptr(dtb), L.ptr(q),
           L.ptr(k), L.ptr(v), L.ptr(conv_out), L.ptr(ops), L.ptr(U), L.ptr(gC), S, L.stream())
    return q, k, v, ops, U, gC


def prep_a(proj, conv_state, conv_w, A_log, dt_bias, relaxed=True):
    """conv+silu+qk-norm and phase A in one launch (qwen35/gdn_nax.py:394-401).
    proj [S,8224], conv_state [3,6144], conv_w [6144,4,1] -> q, k, v [S,16,128] bf16 and the three phase-B records."""
    return _phase_a(proj, conv_state, conv_w, A_log, dt_bias)


def gdn_chunked(q, k, v, proj, A_log, dt_bias, state, relaxed=True, flags=DEFAULT_FLAGS, tg=None):
    """q,k,v [S,16,128] bf16 (q/k already normalized + scaled), proj [S,8224] bf16 (b at 8192:8208, a at 8208:8224),
    state [1,16,128,128] fp32.  Returns y [S,16,128] bf16, new_state [1,16,128,128] fp32  (qwen35/gdn_nax.py:413-426)."""
    _, _, _, ops, U, gC = _phase_a(proj, None, None, A_log, dt_bias, qkv=(q, k, v))
    return phase_b(q, k, v, ops, U, gC, state)


_SNAP = {}            # (device index, stream handle) -> float16 tensor: flag area + chain snapshots
_SNAP_RETIRED = []    # outgrown buffers stay alive: a captured HIP graph may hold their address
_STATUS = {}          # (device index, stream handle) -> pinned int32[1]: the last copy of the buffer's status word

GAVE_UP, NOT_FINITE = 1, 2        # bits of the status word


class ChunkedPrefillError(RuntimeError):
    """A chunked-prefill launch on this stream reported a failure in its status word: its results are not to be used."""


def _key(dev):
    return (dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)


def _snap_buffer(dev, nbytes):
    """The buffer between phase B's chain and output workgroups, cached per (device, stream): its first 33 KiB are the flag
    area, which has to be zero before a launch and is left zero by it, so the buffer is zero-filled once, when it is made."""
    key = _key(dev)
    buf = _SNAP.get(key)
    if buf is None or buf.numel() * 2 < nbytes:
        if buf is not None:
            _raise_if_failed(key, buf, sync=True)          # the old buffer's word is looked at one last time
            _SNAP_RETIRED.append(buf)
        buf = torch.zeros(max(nbytes // 2, 8), dtype=torch.float16, device=dev)
        _SNAP[key] = buf
        _STATUS[key] = torch.zeros(1, dtype=torch.int32, pin_memory=True)
    return buf


def _status_word(buf):
    off = L.lib().qt_gdn_chunk_status_offset() // 4
    return buf.view(torch.int32)[off:off + 1]


def _describe(v):
    what = []
    if v & GAVE_UP:
        what.append("an output workgroup waited for its chunk for too long and gave up (its rows were not written)")
    if v & NOT_FINITE:
        what.append("the final state is not finite: a half-precision operand overflowed (|state|, |v| or an intermediate above 65504)")
    return "; ".join(what) or f"status {v}"


def _raise_if_failed(key, buf, sync=False):
    """Looks at the status word of the launches made so far with `buf`.  Without `sync` it reads the host copy that the last
    launch's asynchronous read-back has left (no wait: a launch still in flight is judged at the next call); with `sync` it
    waits for the stream first.  A set word is cleared on the device and raised as ChunkedPrefillError."""
    pin = _STATUS[key]
    if sync and not torch.cuda.is_current_stream_capturing():
        torch.cuda.current_stream(buf.device).synchronize()
        pin.copy_(_status_word(buf))
    v = int(pin[0])
    if v:
        torch.cuda.current_stream(buf.device).synchronize()     # error path only: no read-back may land after the reset
        _status_word(buf).zero_()
        pin.zero_()
        raise ChunkedPrefillError("chunked prefill: " + _describe(v))


def _read_back_status(key, buf):
    """Enqueues the copy of the status word to pinned host memory behind the launch (skipped under graph capture)."""
    if not torch.cuda.is_current_stream_capturing():
        _STATUS[key].copy_(_status_word(buf), non_blocking=True)


def check_status(device=None, sync=True):
    """Raises ChunkedPrefillError if a chunked-prefill launch on the current stream of `device` has failed (see
    _raise_if_failed).  phase_b / phase_b_norm call this without waiting before every launch, so a failure surfaces at the
    next call at the latest; a caller that needs the answer for the launches already made calls it with sync=True."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    key = _key(dev)
    if key in _SNAP:
        _raise_if_failed(key, _SNAP[key], sync=sync)


def _phase_b_args(S, Tb, Am, gv, state):
    ops, U, gC = L.dev(Tb, torch.float16, "Tb"), L.dev(Am, torch.float16, "Am"), L.dev(gv, torch.float32, "gv")
    lib = L.lib()
    if ops.numel() * 2 < lib.qt_gdn_chunk_ops_bytes(S) or U.numel() * 2 < lib.qt_gdn_chunk_u_bytes(S) or \
            gC.numel() * 4 < lib.qt_gdn_chunk_gc_bytes(S):
        raise ValueError("phase_b: the phase A records are too small for this many tokens")
    state = L.dev(state, torch.float32, "state").reshape(1, HV, DV, DK)
    snap = _snap_buffer(state.device, lib.qt_gdn_chunk_snap_bytes(S))
    _raise_if_failed(_key(state.device), snap)              # the previous launch with this buffer, if its word has arrived
    return ops, U, gC, snap, state, torch.empty_like(state)


def phase_b(q, k, v, Tb, Am, gv, state, relaxed=True, flags=DEFAULT_FLAGS, tg=None):
    """The serial state recurrence on the outputs of phase A -> y [S,16,128] bf16, new state [1,16,128,128] f32
    (qwen35/gdn_nax.py:404-410).  Tb / Am / gv are the records prep_a (or gdn_chunked's phase A) produced."""
    S = q.shape[0]
    ops, U, gC, snap, state, out = _phase_b_args(S, Tb, Am, gv, state)
    y = torch.empty((S, HV, DV), dtype=BF16, device=state.device)
    L.call("qt_gdn_phase_b", L.ptr(ops), L.ptr(U), L.ptr(gC), L.ptr(snap), L.ptr(state), L.ptr(out), L.ptr(y), S, L.stream())
    _read_back_status(_key(state.device), snap)
    return y, out


def phase_b_norm(proj, Tb, Am, gv, state, gw, eps=1e-6):
    """phase_b followed by prefill.gated_norm (qwen35/prefill.py:241-244) in one pass: the outputs never leave the chip
    un-normalised.  proj [S,8224] bf16 supplies z; gw [128].  -> out [S,2048] bf16, new state [1,16,128,128] f32."""
    proj = L.dev(proj, BF16, "proj", (None, PW))
    S = proj.shape[0]
    ops, U, gC, snap, state, new_state = _phase_b_args(S, Tb, Am, gv, state)
    gw = L.f32(gw, "gw", (DV,))
    out = torch.empty((S, HV * DV), dtype=BF16, device=state.device)
    L.call("qt_gdn_phase_b_norm", L.ptr(ops), L.ptr(U), L.ptr(gC), L.ptr(snap), L.ptr(state), L.ptr(new_state), L.ptr(proj),
           L.ptr(gw), float(eps), L.ptr(out), S, L.stream())
    _read_back_status(_key(state.device), snap)
    return out, new_state
