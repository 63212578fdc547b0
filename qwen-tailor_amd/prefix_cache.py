"""Checkpoints of the path's state for resuming a prefill from a token prefix seen before (qwen35/prefix_cache.py).

A checkpoint (node) is the complete recurrent state after `pos` tokens -- ssm [18, 1, 16, 128, 128] float32 and conv
[18, 1, 3, 6144] bf16 -- plus the K / V rows [parent.pos : pos) of the 6 full-attention layers as one segment
kv [12, 1, 2, pos - parent.pos, 256] bf16 (K and V of a layer interleaved), the tokens themselves and optional extras
(qwen35/prefix_cache.py:31-46, 173-188).  `lookup` finds the deepest checkpoint that is a prefix of a new prompt, `restore`
concatenates the chain's segments into fresh contiguous K / V buffers, eviction drops least recently used leaves.

The bookkeeping is host Python, as in the reference.  Every byte of state moves through the strided copy kernel (one
`blit_batch` launch per checkpoint / restore).  torch tensors are mutable, so where the reference shares the immutable
recurrent arrays with the restored state (qwen35/prefix_cache.py:136-137), `restore` hands out copies: decoding from a
restored state must never write into the cache.
"""
from __future__ import annotations

import numpy as np
import torch

from .batch import blit_batch

BF16 = torch.bfloat16


class Node:
    """One checkpoint: `pos` tokens (`toks`), the recurrent state after them (`conv`, `ssm`), the K / V rows since the parent
    checkpoint (`kv`), what an exact repeat of the prompt needs (`last`), engine extras (`extra`) and the cache's own
    bookkeeping (`nbytes`, `stamp` of last use, `nchild`, `uid`).  Field names as qwen35/prefix_cache.py:31-46."""
    __slots__ = ("parent", "pos", "toks", "kv", "conv", "ssm", "last", "extra", "nbytes", "stamp", "nchild", "uid")

    def __init__(self, parent=None, pos=0, toks=None):
        self.parent, self.pos, self.toks = parent, pos, toks
        self.kv = self.conv = self.ssm = self.last = self.extra = None
        self.nbytes = self.stamp = self.nchild = self.uid = 0

    def chain(self):
        """the checkpoints from the root down to this one"""
        up = [self]
        while up[-1].parent is not None:
            up.append(up[-1].parent)
        return up[::-1]


def _size(values):
    """bytes held by the tensors / arrays among `values`"""
    total = 0
    for v in values:
        if isinstance(v, torch.Tensor):
            total += v.numel() * v.element_size()
        elif isinstance(v, np.ndarray):
            total += v.nbytes
    return total


def _detach(d):
    """A dict whose tensors own their storage: a view (the last hidden row of a big activation) would keep the whole activation
    alive for as long as the entry lives (qwen35/prefix_cache.py:49-52)."""
    if d is None:
        return None
    return {k: v.clone() if isinstance(v, torch.Tensor) else v for k, v in d.items()}


def common_prefix(a, b):
    """length of the longest common prefix of two int arrays"""
    n = min(len(a), len(b))
    differ = np.flatnonzero(a[:n] != b[:n])
    return int(differ[0]) if differ.size else n


class PrefixCache:
    # thresholds of split learning, in tokens (values of qwen35/prefix_cache.py:58-59): the common prefix of two prompts becomes a
    # checkpoint only if it is at least MIN_SPLIT long and reaches at least MIN_GAIN past the checkpoint a lookup already hits
    MIN_SPLIT = 32
    MIN_GAIN = 32

    def __init__(self, budget_mb=1024):
        self.budget = int(budget_mb * (1 << 20))
        self.nodes: dict[int, Node] = {}       # uid -> checkpoint
        self._index: dict[tuple, int] = {}     # (pos, token bytes) -> uid: an identical prompt prefix is stored once
        self.bytes = 0
        self._clock = 0
        self._uid = 0
        self.stats = dict.fromkeys(("lookups", "hits", "hit_tokens", "prompt_tokens", "inserted", "evicted", "splits"), 0)
        self.last_hit = 0                      # pos of the checkpoint used by the latest lookup (0 = miss)
        self._zeros = None                     # a block of zero rows on the device, the source of the padding in restore

    def __len__(self):
        return len(self.nodes)

    def _touch(self, node):
        """mark the whole chain of `node` as used now"""
        self._clock += 1
        for c in node.chain():
            c.stamp = self._clock

    # ---- lookup (qwen35/prefix_cache.py:90-125) ---------------------------------------------------------------------
    def lookup(self, ids):
        """ids: token ids of the new prompt.  Returns (node, split): the deepest checkpoint that is a prefix of ids (None =
        miss; a checkpoint that covers the whole prompt only counts if it carries `last`), and a position (0 = none) at
        which the new prefill should add a checkpoint because the prompt overlaps a stored one up to there."""
        prompt = np.asarray(ids, dtype=np.int32)
        S = len(prompt)
        hit, overlap = None, 0
        for nd in self.nodes.values():
            shared = common_prefix(nd.toks, prompt)
            if shared < nd.pos:                                  # parts ways with the prompt before the checkpoint ...
                if shared < S:                                   # ... and inside the prompt: a place for a new checkpoint
                    overlap = max(overlap, shared)
            elif (nd.pos < S or nd.last is not None) and (hit is None or nd.pos > hit.pos):
                hit = nd
        base = 0 if hit is None else hit.pos
        split = overlap if overlap >= self.MIN_SPLIT and overlap - base >= self.MIN_GAIN else 0
        self.stats["lookups"] += 1
        self.stats["prompt_tokens"] += S
        self.stats["hits"] += hit is not None
        self.stats["hit_tokens"] += base
        self.stats["splits"] += split > 0
        self.last_hit = base
        if hit is not None:
            self._touch(hit)
        return hit, split

    # ---- the device copies ------------------------------------------------------------------------------------------
    @staticmethod
    def _snapshot(state, a, pos):
        """(kv [12,1,2,pos-a,256], conv [18,1,3,6144], ssm [18,1,16,128,128]) copied out of the live state in one launch"""
        kvs = [x for k, v in state["kv"] for x in (k, v)]
        dev = kvs[0].device
        nkv, D, n = kvs[0].shape[1], kvs[0].shape[3], pos - a
        kv = torch.empty((len(kvs), 1, nkv, n, D), dtype=BF16, device=dev)
        conv = torch.empty((len(state["conv"]),) + tuple(state["conv"][0].shape), dtype=BF16, device=dev)
        ssm = torch.empty((len(state["ssm"]),) + tuple(state["ssm"][0].shape), dtype=torch.float32, device=dev)
        jobs = []
        for j, x in enumerate(kvs):                              # rows [a, pos) of both KV heads
            L = x.shape[2]
            jobs.append((kv, x, n * D, j * nkv * n * D, a * D, nkv, n * D, L * D))
        for i, c in enumerate(state["conv"]):
            jobs.append((conv, c, c.numel(), i * c.numel(), 0, 1, 0, 0))
        for i, s in enumerate(state["ssm"]):
            jobs.append((ssm, s, s.numel(), i * s.numel(), 0, 1, 0, 0))
        blit_batch(jobs)
        return kv, conv, ssm

    @staticmethod
    def cat_rows(chain, get, total, axis):
        """The segments `get(node)` of the nodes of `chain` (tensors that differ along `axis` only; None = the node has none)
        laid end to end along `axis` in one tensor of `total` rows, the rows past the last segment zero (the role of
        qwen35/prefix_cache.py:124-132; the owning engine uses it for its `extra` segments).  At least one node must have a segment."""
        segs = [t for t in map(get, chain) if t is not None]
        first = segs[0]
        shape = list(first.shape)
        shape[axis] = max(total, sum(t.shape[axis] for t in segs))
        if len(segs) == 1 and shape[axis] == first.shape[axis]:
            return first
        out = torch.zeros(shape, dtype=first.dtype, device=first.device)
        at = 0
        for t in segs:
            out.narrow(axis, at, t.shape[axis]).copy_(t)
            at += t.shape[axis]
        return out

    def restore(self, node, max_len):
        """(state, chain): the state dict of the checkpoint ({"kv": [(K, V)] x6 [1,2,max_len,256], "conv": [...], "ssm": [...]}),
        all tensors fresh: K / V rows [0, pos) are the chain's segments end to end, rows [pos, max_len) are zero
        (qwen35/prefix_cache.py:139-154)."""
        assert node.pos <= max_len, (node.pos, max_len)
        chain = node.chain()
        nb, _, nkv, _, D = node.kv.shape
        dev = node.kv.device
        bufs = [torch.empty((1, nkv, max_len, D), dtype=BF16, device=dev) for _ in range(nb)]
        conv = [torch.empty_like(node.conv[i]) for i in range(node.conv.shape[0])]
        ssm = [torch.empty_like(node.ssm[i]) for i in range(node.ssm.shape[0])]
        jobs, a = [], 0
        for c in chain:
            n = c.kv.shape[3]
            for j in range(nb):
                jobs.append((bufs[j], c.kv, n * D, a * D, j * nkv * n * D, nkv, max_len * D, n * D))
            a += n
        assert a == node.pos, (a, node.pos)
        for i in range(len(conv)):
            jobs.append((conv[i], node.conv, conv[i].numel(), 0, i * conv[i].numel(), 1, 0, 0))
        for i in range(len(ssm)):
            jobs.append((ssm[i], node.ssm, ssm[i].numel(), 0, i * ssm[i].numel(), 1, 0, 0))
        if max_len > node.pos:                                   # rows [pos, max_len) from a block of zeros, in the same launch
            pad = (max_len - node.pos) * D
            if self._zeros is None or self._zeros.numel() < pad or self._zeros.device != dev:
                self._zeros = torch.zeros(pad, dtype=BF16, device=dev)
            for b in bufs:
                jobs.append((b, self._zeros, pad, node.pos * D, 0, nkv, max_len * D, 0))
        blit_batch(jobs)
        st = {"kv": [(bufs[2 * i], bufs[2 * i + 1]) for i in range(nb // 2)], "conv": conv, "ssm": ssm}
        return st, chain

    # ---- insert / evict (qwen35/prefix_cache.py:157-218) ------------------------------------------------------------
    def insert(self, parent, toks, pos, state, last=None, extra=None):
        """Checkpoint the live `state` (valid after `pos` tokens; K / V rows [parent.pos : pos) are the new ones).  `toks`: the
        prompt's token ids (>= pos long).  `last`: optional dict with what a hit at pos == len(prompt) needs; `extra`: dict of
        per-segment tensors for the owning engine.  Returns the node (an existing one for identical tokens; `parent` if the
        checkpoint alone exceeds the budget)."""
        toks = np.ascontiguousarray(np.asarray(toks, dtype=np.int32)[:pos])
        key = (pos, toks.tobytes())
        known = self.nodes.get(self._index.get(key, -1))
        if known is not None:
            self._touch(known)
            if known.last is None and last is not None:          # the repeat brings what a whole-prompt hit needs
                known.last = _detach(last)
                grow = _size(known.last.values())
                known.nbytes += grow
                self.bytes += grow
            return known
        start = 0 if parent is None else parent.pos
        assert pos > start, (pos, start)
        nd = Node(parent, pos, toks.copy())
        nd.kv, nd.conv, nd.ssm = self._snapshot(state, start, pos)
        nd.last, nd.extra = _detach(last), extra
        nd.nbytes = _size([nd.kv, nd.conv, nd.ssm]) + _size((nd.last or {}).values()) + _size((extra or {}).values())
        if nd.nbytes > self.budget:
            return parent
        self._uid += 1
        nd.uid = self._uid
        self.nodes[nd.uid] = nd
        self._index[key] = nd.uid
        if parent is not None:
            parent.nchild += 1
        self.bytes += nd.nbytes
        self.stats["inserted"] += 1
        self._touch(nd)
        self._evict(protect=nd)
        return nd

    def _evict(self, protect=None):
        """drop least recently used leaves until the budget holds; the chain of `protect` (being built or used) stays"""
        pinned = {c.uid for c in protect.chain()} if protect is not None else set()
        while self.bytes > self.budget:
            leaves = [n for n in self.nodes.values() if not n.nchild and n.uid not in pinned]
            if not leaves:
                return
            victim = min(leaves, key=lambda n: n.stamp)
            self.nodes.pop(victim.uid)
            self._index.pop((victim.pos, victim.toks.tobytes()), None)
            if victim.parent is not None:
                victim.parent.nchild -= 1
            self.bytes -= victim.nbytes
            self.stats["evicted"] += 1

    def clear(self):
        self.nodes.clear()
        self._index.clear()
        self.bytes = 0
