"""Batched speculative verify: the GatedDeltaNet part of qwen35/batch_spec.py (deltanet_bm, SpecPools)."""
from __future__ import annotations

import torch

from . import _lib as L
from .kernels import flat_conv_w
from .model import Cfg

BF16 = torch.bfloat16
HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224


def deltanet_bm(proj, conv_pool, conv_w, A_log, dt_bias, ssm_pool, sslots, sels, pars, M, rows_per_wg: int = 0):
    """proj [B*M, 8224] bf16 (row b*M+j = token j of sequence b); sslots / sels / pars int32 [B]: the sequence's entry in the
    snapshot pools, the snapshot it starts from, and the conv buffer it reads.  Returns y [B*M, 2048] bf16; writes snapshots
    0..M-1 of ssm_pool[sslot] and conv buffer par^1 IN PLACE (qwen35/batch_spec.py:142-150)."""
    sslots = L.i32(sslots, "sslots")
    B = sslots.shape[0]
    proj = L.dev(proj, BF16, "proj", (B * M, PW))
    ssm_pool = L.dev(ssm_pool, torch.float32, "ssm_pool", (None, M, HV, DV, DK))
    n_entries = ssm_pool.shape[0]
    conv_pool = L.dev(conv_pool, BF16, "conv_pool", (n_entries * 2, M, 3, CD))
    sels, pars = L.i32(sels, "sels", B), L.i32(pars, "pars", B)
    w = flat_conv_w(conv_w)
    A, dtb = L.f32(A_log, "A_log", (HV,)), L.f32(dt_bias, "dt_bias", (HV,))
    y = torch.empty((B * M, HV * DV), dtype=BF16, device=proj.device)
    L.call("qt_gdn_verify_step", L.ptr(proj), L.ptr(conv_pool), L.ptr(w), L.ptr(A), L.ptr(dtb), L.ptr(ssm_pool), L.ptr(sslots),
           L.ptr(sels), L.ptr(pars), L.ptr(y), B, M, n_entries, rows_per_wg, L.stream())
    return y


class SpecPools:
    """Snapshot pools of the sequences in speculative mode (qwen35/batch_spec.py:242-270; the recurrent part and the K / V
    pool of the draft layer)."""

    def __init__(self, cfg: Cfg, nspec: int, nslots: int, M: int, max_len: int, device="cuda"):
        self.cfg, self.NS, self.M, self.Lmax = cfg, nspec, M, max_len
        nl = sum(cfg.is_linear(i) for i in range(cfg.layers))
        z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=device)
        self.conv = [z(((nspec + 1) * 2, M, 3, CD), BF16) for _ in range(nl)]
        self.ssm = [z((nspec + 1, M, HV, DV, DK), torch.float32) for _ in range(nl)]
        self.mK = z((nslots + 1, cfg.n_kv, max_len, cfg.head_dim), BF16)
        self.mV = z((nslots + 1, cfg.n_kv, max_len, cfg.head_dim), BF16)

    def as_tree(self):
        return {"conv": self.conv, "ssm": self.ssm, "mK": self.mK, "mV": self.mV}

    @staticmethod
    def entry_bytes(cfg: Cfg, M: int):
        nl = sum(cfg.is_linear(i) for i in range(cfg.layers))
        return nl * M * (HV * DV * DK * 4 + 2 * 3 * CD * 2)


def to_spec(P, SP, slot: int, pos: int, ss: int):
    """Plain -> speculative (the state moves of qwen35/serve.py:310-330): the sequence in `slot` of the plain pools `P`, with
    `pos` tokens in its state, goes into snapshot 0 / conv buffer 0 of entry `ss` of the snapshot pools `SP`, for every
    GatedDeltaNet layer.  The caller then runs the entry with par = 0, sel = 0."""
    from .batch import blit_batch
    M = SP.M
    jobs = []
    for i in range(len(SP.conv)):
        jobs.append((SP.conv[i], P.conv[i], 3 * CD, (ss * 2 * M) * 3 * CD, (slot * 2 + (pos & 1)) * 3 * CD, 1, 0, 0))
        jobs.append((SP.ssm[i], P.ssm[i], HV * DV * DK, ss * M * HV * DV * DK, slot * HV * DV * DK, 1, 0, 0))
    blit_batch(jobs)


def to_plain(P, SP, slot: int, pos: int, ss: int, par: int, n: int):
    """Speculative -> plain (qwen35/serve.py:332-348): the live snapshot `n` of entry `ss` (conv buffer `par`, the one the
    last round wrote) goes back into `slot` of the plain pools, whose state then holds `pos` tokens."""
    from .batch import blit_batch
    M = SP.M
    jobs = []
    for i in range(len(SP.conv)):
        jobs.append((P.ssm[i], SP.ssm[i], HV * DV * DK, slot * HV * DV * DK, (ss * M + n) * HV * DV * DK, 1, 0, 0))
        jobs.append((P.conv[i], SP.conv[i], 3 * CD, (slot * 2 + (pos & 1)) * 3 * CD, ((ss * 2 + par) * M + n) * 3 * CD, 1, 0, 0))
    blit_batch(jobs)
