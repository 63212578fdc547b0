"""GPU parity of the prefix-cache checkpoints (qwen35/prefix_cache.py:139-188): the K / V segments, the stacked recurrent state
and the restored buffers against the numpy restatement, bit exact; a restored state never aliases the cache; the chain
prefill -> checkpoint -> restore -> admission into the slot pools returns the state bit for bit."""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    q._lib.lib()
    return q


def make_state(qt, dev, max_len, seed):
    cfg = qt.model.Cfg()
    nl = sum(cfg.is_linear(i) for i in range(cfg.layers))
    na = cfg.layers - nl
    g = torch.Generator().manual_seed(seed)
    r = lambda shape, dt: torch.randn(shape, generator=g).to(dt).to(dev)
    return cfg, {"kv": [(r((1, cfg.n_kv, max_len, cfg.head_dim), BF16), r((1, cfg.n_kv, max_len, cfg.head_dim), BF16)) for _ in range(na)],
                 "conv": [r((1, 3, CD), BF16) for _ in range(nl)], "ssm": [r((1, HV, DV, DK), torch.float32) for _ in range(nl)]}


def test_checkpoint_chain_and_restore_bit_exact(qt, dev):
    cfg, st = make_state(qt, dev, 96, 1)
    kv_np = [(to_np(k), to_np(v)) for k, v in st["kv"]]
    toks = np.arange(200, dtype=np.int32)
    pc = qt.prefix_cache.PrefixCache(budget_mb=512)
    n1 = pc.insert(None, toks, 40, st)
    check_equal("segment 0..40", to_np(n1.kv), O.pc_segment(kv_np, 0, 40))
    assert tuple(n1.conv.shape) == (len(st["conv"]), 1, 3, CD) and tuple(n1.ssm.shape) == (len(st["ssm"]), 1, HV, DV, DK)
    for i in range(len(st["conv"])):
        assert torch.equal(n1.conv[i], st["conv"][i]) and torch.equal(n1.ssm[i], st["ssm"][i])
    conv1 = [c.clone() for c in st["conv"]]
    for c, s in zip(st["conv"], st["ssm"]):                                    # the prefill moves on: the recurrent state changes in place
        c.add_(1.0)
        s.mul_(0.5)
    n2 = pc.insert(n1, toks, 77, st, last={"tok": 3})
    check_equal("segment 40..77", to_np(n2.kv), O.pc_segment(kv_np, 40, 77))
    assert n1.nbytes == n1.kv.numel() * 2 + n1.conv.numel() * 2 + n1.ssm.numel() * 4 and pc.bytes == n1.nbytes + n2.nbytes
    assert all(torch.equal(n1.conv[i], conv1[i]) for i in range(len(conv1)))   # the first checkpoint kept its own copy

    got, chain = pc.restore(n2, 128)
    assert chain == [n1, n2]
    want = O.pc_restore([to_np(n1.kv), to_np(n2.kv)], 128)
    for (gk, gv), (wk, wv), (sk, sv) in zip(got["kv"], want, kv_np):
        check_equal("restored K", to_np(gk), wk)
        check_equal("restored V", to_np(gv), wv)
        assert np.array_equal(to_np(gk)[:, :, :77], sk[:, :, :77]) and not to_np(gv)[:, :, 77:].any()
    for i in range(len(st["conv"])):
        assert torch.equal(got["conv"][i], st["conv"][i]) and torch.equal(got["ssm"][i], st["ssm"][i])

    got["ssm"][0].zero_()                                                      # decoding from a restored state writes in place ...
    got["kv"][0][0].zero_()
    again, _ = pc.restore(n2, 128)
    assert torch.equal(again["ssm"][0], st["ssm"][0]) and np.array_equal(to_np(again["kv"][0][0])[:, :, :77], kv_np[0][0][:, :, :77])

    only, chain1 = pc.restore(n1, 40)                                          # max_len == pos: no padding rows
    assert chain1 == [n1] and tuple(only["kv"][0][0].shape) == (1, cfg.n_kv, 40, cfg.head_dim)
    check_equal("restore without pad", to_np(only["kv"][2][1]), kv_np[2][1][:, :, :40])
    hit, split = pc.lookup(toks[:77])
    assert hit is n2 and split == 0


def test_restore_then_admission_into_slot_pools(qt, dev):
    """the resume path end to end: checkpoint, restore, Pools.load, Pools.read"""
    cfg, st = make_state(qt, dev, 64, 2)
    pc = qt.prefix_cache.PrefixCache(budget_mb=512)
    node = pc.insert(None, np.arange(64, dtype=np.int32), 51, st)
    restored, _ = pc.restore(node, 64)
    P = qt.batch.Pools(cfg, 2, 80, device=dev)
    P.load(1, restored, 51)
    back = P.read(1, 51, 64)
    for (k, v), (k0, v0) in zip(back["kv"], st["kv"]):
        assert torch.equal(k[:, :, :51], k0[:, :, :51]) and torch.equal(v[:, :, :51], v0[:, :, :51])
    for i in range(len(st["conv"])):
        assert torch.equal(back["conv"][i], st["conv"][i]) and torch.equal(back["ssm"][i], st["ssm"][i])


def test_cat_rows_pads_with_zeros(qt, dev):
    pc = qt.prefix_cache.PrefixCache
    a, b = torch.ones((1, 3, 4), device=dev), 2 * torch.ones((1, 5, 4), device=dev)

    class N:
        def __init__(self, x):
            self.x = x
    out = pc.cat_rows([N(a), N(None), N(b)], lambda n: n.x, 10, 1)
    assert tuple(out.shape) == (1, 10, 4) and out[0, :3].eq(1).all() and out[0, 3:8].eq(2).all() and not out[0, 8:].any()
