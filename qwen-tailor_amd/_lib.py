"""ctypes binding of csrc/libqwen_tailor_hip.so (the C ABI declared in include/qwen_tailor_hip.h).

There is no CPU fallback: every operator of this package runs a HIP kernel or raises."""
from __future__ import annotations

import ctypes
import os

import torch

from . import _build

_lib = None
_vp, _i, _l, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

ERRORS = {-1: "bad dimension", -2: "misaligned pointer", -3: "null pointer", -4: "unsupported shape", -5: "kernel launch failed",
          -6: "workspace too small", -7: "size beyond the maximum of the allocation-free entry point"}

_SIGS = {
    "qt_gdn_decode_step": [_vp] * 9 + [_i, _i, _i, _vp],
    "qt_gdn_decode_step_gnorm": [_vp] * 9 + [_f, _vp, _i, _i, _vp],
    "qt_gdn_verify_step": [_vp] * 10 + [_i, _i, _i, _i, _vp],
    "qt_gdn_deltanet": [_vp] * 10 + [_i, _i, _i, _vp],
    "qt_gdn_gates": [_vp, _vp, _l, _l, _vp, _vp, _vp, _vp, _vp, _l, _i, _vp],
    "qt_normalize_qk": [_vp, _vp, _vp, _vp, _l, _i, _vp],
    "qt_gdn_conv_prep": [_vp] * 7 + [_i, _vp],
    "qt_silu_table_build": [_vp, _vp],
    "qt_gated_rmsnorm": [_vp, _vp, _vp, _vp, _l, _f, _vp],
    "qt_gdn_recurrent": [_vp] * 8 + [_i] * 6 + [_vp],
    "qt_gqa_attn_decode": [_vp] * 9 + [_l, _i, _i, _i, _i, _i, _vp],
    "qt_gqa_attn_decode_static": [_vp] * 8 + [_i, _i, _i, _i, _i, _vp],
    "qt_gqa_attn_layer_decode": [_vp] * 4 + [_i] + [_vp] * 6 + [_l, _i, _i, _i, _i, _i, _f, _vp],
    "qt_rope_table_build": [_vp, _i, _vp],
    "qt_gdn_phase_b": [_vp] * 7 + [_i, _vp],
    "qt_gdn_phase_b_poll_limit": [_i],
    "qt_gdn_phase_b_norm": [_vp] * 8 + [_f, _vp, _i, _vp],
    "qt_gqa_prefill_causal": [_vp] * 5 + [_l, _i, _i, _i, _l, _l, _vp],
    "qt_gdn_phase_a": [_vp] * 9 + [_i, _vp],
    "qt_gdn_phase_a_conv": [_vp] * 13 + [_i, _vp],
    "qt_blit": [_vp, _vp, _i, _l, _l, _l, _l, _l, _l, _vp],
    "qt_attn_qkv_prep": [_vp] * 7 + [_l, _i, _f, _vp],
    "qt_attn_qkv_prep_table": [_vp] * 5 + [_i] + [_vp] * 3 + [_l, _i, _f, _vp],
    "qt_attn_out_gate": [_vp, _vp, _vp, _l, _vp],
    "qt_blit_batch": [_vp, _vp, _vp, _i, _vp],
    "qt_rms_rows": [_vp, _vp, _vp, _i, _i, _f, _vp],
    "qt_fused_gemv": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
}


def lib():
    """The loaded library.  Builds it first if no built library is present or if it was built from other sources than the
    ones in csrc/ now (a hash of the sources is stored beside it); raises if that is impossible."""
    global _lib
    if _lib is None:
        if not _build.is_current():
            _build.build()
        L = ctypes.CDLL(_build.SO)
        for name, args in _SIGS.items():
            fn = getattr(L, name)
            fn.argtypes, fn.restype = args, ctypes.c_int
        L.qt_gqa_attn_workspace_bytes.argtypes, L.qt_gqa_attn_workspace_bytes.restype = [_i] * 4, ctypes.c_long
        L.qt_gdn_chunk_status_offset.argtypes, L.qt_gdn_chunk_status_offset.restype = [], ctypes.c_long
        L.qt_rope_table_bytes.argtypes, L.qt_rope_table_bytes.restype = [_i], ctypes.c_long
        for name in ("qt_gdn_chunk_ops_bytes", "qt_gdn_chunk_u_bytes", "qt_gdn_chunk_gc_bytes", "qt_gdn_chunk_snap_bytes",
                     "qt_gqa_prefill_workspace_bytes"):
            getattr(L, name).argtypes, getattr(L, name).restype = [_i], ctypes.c_long
        L.qt_gqa_prefill_workspace_bytes_for.argtypes, L.qt_gqa_prefill_workspace_bytes_for.restype = [_i] * 3, ctypes.c_long
        _lib = L
    return _lib


def declare(name, args):
    """Register the signature of one more entry point (used by the modules that own it)."""
    _SIGS[name] = args
    if _lib is not None:
        fn = getattr(_lib, name)
        fn.argtypes, fn.restype = args, ctypes.c_int


def call(name, *args):
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed: {ERRORS.get(rc, rc)}")


_SILU_TABLES = {}


def silu_table(dev):
    """The 11 KiB silu_bf16 table of `dev` (built once per device by the library, owned here: the C ABI keeps no state)."""
    t = _SILU_TABLES.get(dev)
    if t is None:
        t = torch.empty(lib().qt_silu_table_bytes() // 2, dtype=torch.bfloat16, device=dev)
        call("qt_silu_table_build", ptr(t), stream())
        _SILU_TABLES[dev] = t
    return t


_ROPE_TABLES = {}        # device -> float32 [positions, 32, 2]
_ROPE_RETIRED = []       # outgrown tables stay alive: a captured HIP graph may hold their address


def rope_table(dev, n_pos):
    """The (cos, sin) pairs of the rotary embedding for positions 0 .. n_pos - 1 on `dev` (built by the library, owned here;
    grown in steps of 16384 positions).  Returns (tensor, positions it covers)."""
    t = _ROPE_TABLES.get(dev)
    if t is None or t.shape[0] < n_pos:
        if t is not None:
            _ROPE_RETIRED.append(t)
        n = -(-max(n_pos, 1) // 16384) * 16384
        t = torch.empty((n, 32, 2), dtype=torch.float32, device=dev)
        call("qt_rope_table_build", ptr(t), n, stream())
        _ROPE_TABLES[dev] = t
    return t, t.shape[0]


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


_WORKSPACES = {}         # (purpose, device index, stream handle) -> uint8 tensor
_RETIRED = []            # outgrown buffers: kept for the life of the process, a captured HIP graph may still hold their address


def workspace(purpose, dev, nbytes, first_bytes=0):
    """Scratch memory for a kernel's partial results (the C ABI never allocates): one uint8 buffer per (purpose, device, stream),
    because launches on different streams may overlap.  A buffer that is outgrown is replaced but never freed: a HIP graph
    captured earlier replays with the old address.  first_bytes: size of the first allocation, so that growth is rare."""
    key = (purpose, dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _RETIRED.append(buf)
        buf = torch.empty(max(nbytes, first_bytes), dtype=torch.uint8, device=dev)
        _WORKSPACES[key] = buf
    return buf


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def dev(t, dtype, name, shape=None):
    """Check that `t` is a contiguous device tensor of `dtype` (and of `shape`, None entries free); return it."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name}: expected a tensor on the GPU")
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    if shape is not None:
        if t.dim() != len(shape) or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise ValueError(f"{name}: expected shape {shape}, got {tuple(t.shape)}")
    return t


def f32(t, name, shape=None):
    """Per-head parameter vectors (A_log, dt_bias, norm weight) are consumed as float32."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name}: expected a tensor on the GPU")
    if t.dtype != torch.float32 or not t.is_contiguous():
        t = t.float().contiguous()
    return dev(t, torch.float32, name, shape)


def i32(t, name, n=None):
    return dev(t, torch.int32, name, None if n is None else (n,))
