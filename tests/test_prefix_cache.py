"""Prefix-cache checkpoints (qwen35/prefix_cache.py): the host bookkeeping on the CPU (lookup rule against a plain-loop
restatement, duplicate detection, byte accounting, least-recently-used eviction), with the device copies replaced by a stand-in;
the copies themselves are checked on the GPU in tests/test_prefix_cache_gpu.py."""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O


def make_cache(budget_mb=1.0, node_bytes=1 << 18):
    import qwen_tailor_amd as qt

    class HostOnly(qt.prefix_cache.PrefixCache):                               # no GPU here: the snapshot is a byte count
        @staticmethod
        def _snapshot(state, a, pos):
            return torch.zeros(node_bytes // 2, dtype=torch.bfloat16), torch.zeros(0, dtype=torch.bfloat16), torch.zeros(0)
    return HostOnly(budget_mb)


def test_oracle_segment_and_restore_by_loops():
    rng = np.random.default_rng(0)
    kv = [(rng.standard_normal((1, 2, 9, 4)).astype(np.float32), rng.standard_normal((1, 2, 9, 4)).astype(np.float32)) for _ in range(3)]
    s1, s2 = O.pc_segment(kv, 0, 4), O.pc_segment(kv, 4, 7)
    assert s1.shape == (6, 1, 2, 4, 4) and s2.shape == (6, 1, 2, 3, 4)
    for j in range(6):
        for h in range(2):
            for r in range(3):
                assert np.array_equal(s2[j, 0, h, r], kv[j // 2][j % 2][0, h, 4 + r])
    out = O.pc_restore([s1, s2], 12)
    for i in range(3):
        for x, src in zip(out[i], kv[i]):
            assert x.shape == (1, 2, 12, 4) and np.array_equal(x[:, :, :7], src[:, :, :7]) and not x[:, :, 7:].any()


def test_lookup_rule_cases():
    pc = make_cache(64)
    A = np.arange(100, dtype=np.int32)
    n40 = pc.insert(None, A, 40, None)
    n70 = pc.insert(n40, A, 70, None, last={"tok": 5})
    assert pc.lookup(A[:90])[0] is n70 and pc.last_hit == 70                  # deepest prefix
    assert pc.lookup(A[:70])[0] is n70                                         # whole prompt: counts because it carries `last`
    assert pc.lookup(A[:40])[0] is None                                        # whole prompt without `last`: no hit
    assert pc.lookup(A[:55])[0] is n40
    B = A.copy()
    B[60] = -1                                                                 # parts ways with the 70-checkpoint at 60
    node, split = pc.lookup(B[:90])
    assert node is n40 and split == 0                                          # 60 - 40 < MIN_GAIN
    C = A.copy()
    C[36] = -1
    assert pc.lookup(C[:90]) == (None, 36)                                     # no hit; a checkpoint at the shared 36 tokens pays
    D = A.copy()
    D[20] = -1
    assert pc.lookup(D[:90]) == (None, 0)                                      # shorter than MIN_SPLIT
    assert pc.stats["lookups"] == 7 and pc.stats["hits"] == 4 and pc.stats["splits"] == 1
    assert pc.stats["hit_tokens"] == 70 + 70 + 40 + 40


def test_lookup_matches_plain_loop_restatement_on_random_trees():
    rng = np.random.default_rng(3)
    for trial in range(30):
        pc = make_cache(64)
        base = rng.integers(0, 3, 200).astype(np.int32)                        # tiny alphabet: many shared prefixes
        nodes, parents = [], [None]
        for _ in range(6):
            par = parents[rng.integers(len(parents))]
            start = 0 if par is None else par.pos
            pos = start + int(rng.integers(1, 60))
            toks = base.copy() if par is None else np.concatenate([par.toks, base[par.pos:]])
            if rng.random() < 0.5:
                toks[start + int(rng.integers(0, pos - start)):] = rng.integers(0, 3, 1)[0]     # a branch of its own
                if par is not None:
                    toks[:par.pos] = par.toks
            last = {"t": 1} if rng.random() < 0.3 else None
            nd = pc.insert(par, toks, pos, None, last=last)
            parents.append(nd)
        listed = list(pc.nodes.values())
        for _ in range(20):
            q = base.copy()
            cut = int(rng.integers(1, 200))
            if rng.random() < 0.7:
                q[int(rng.integers(0, cut)):] = rng.integers(0, 3, 1)[0]
            q = q[:cut]
            got, split = pc.lookup(q)
            wi, wsplit = O.pc_lookup([(n.toks, n.last is not None) for n in listed], q, pc.MIN_SPLIT, pc.MIN_GAIN)
            want = None if wi is None else listed[wi]
            assert (got.pos if got else 0) == (want.pos if want else 0) and split == wsplit


def test_insert_twice_returns_the_same_node_and_adopts_last():
    pc = make_cache(64)
    A = np.arange(50, dtype=np.int32)
    n = pc.insert(None, A, 30, None)
    before = pc.bytes
    again = pc.insert(None, A, 30, None, last={"h": torch.zeros(8)})
    assert again is n and len(pc) == 1 and n.last is not None and pc.bytes == before + 32 and n.nbytes == before + 32
    other = pc.insert(None, np.arange(1, 51, dtype=np.int32), 30, None)
    assert other is not n and len(pc) == 2


def test_eviction_is_lru_over_leaves_and_spares_the_active_chain():
    pc = make_cache(budget_mb=1.0, node_bytes=1 << 18)                         # four nodes fit
    A = np.arange(400, dtype=np.int32)
    a = pc.insert(None, A, 50, None)
    b = pc.insert(a, A, 100, None)
    other = [pc.insert(None, A + 1000 * (i + 1), 50, None) for i in range(2)]
    assert len(pc) == 4 and pc.bytes == 4 << 18
    pc.lookup(np.concatenate([other[0].toks, [7]]))                            # other[0] used last; other[1] is now the oldest leaf
    c = pc.insert(b, A, 150, None)                                             # over budget: the oldest unprotected leaf goes
    assert len(pc) == 4 and other[1].uid not in pc.nodes and pc.stats["evicted"] == 1
    assert all(n.uid in pc.nodes for n in (a, b, c, other[0]))                 # a and b are inner nodes of the chain being built
    assert a.nchild == 1 and b.nchild == 1 and pc.bytes <= pc.budget
    pc.insert(None, A + 9000, 50, None)
    assert other[0].uid not in pc.nodes                                        # next oldest leaf (c was just used)
    assert pc.insert(None, A + 5000, 60, None) is not None and pc.bytes <= pc.budget
    big = make_cache(budget_mb=0.1, node_bytes=1 << 18)
    assert big.insert(None, A, 10, None) is None and len(big) == 0             # a checkpoint larger than the budget is not kept
    pc.clear()
    assert len(pc) == 0 and pc.bytes == 0
