"""GPU parity of the state admission / migration copies (qwen35/batch.py:349-372, 431-462; qwen35/serve.py:310-348) against the
numpy restatement: bit exact, nothing outside the destination ranges touched."""
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,d0,s0,ny,dstride,sstride", [
    (0, 0, 0, 1, 0, 0), (1, 0, 0, 1, 0, 0), (7, 3, 5, 1, 0, 0), (8, 8, 16, 3, 64, 40), (256, 0, 0, 2, 1000, 512),
    (1000, 24, 8, 4, 2048, 1024), (1001, 24, 8, 4, 2048, 1024), (4096, 4096, 0, 1, 0, 0), (18432, 36864, 18432, 1, 0, 0),
    (5000, 16, 32, 2, 8200 * 8, 5008)])
def test_blit_vs_numpy(qt, dev, dtype, n, d0, s0, ny, dstride, sstride):
    rng = np.random.default_rng(n + 7 * ny)
    nd = d0 + (ny - 1) * dstride + n + 13
    ns = s0 + (ny - 1) * sstride + n + 5
    dst0, src = bf(rng.standard_normal(nd)), bf(rng.standard_normal(ns))
    d = to_dev(dst0, dev, dtype)
    qt.batch.blit(d, to_dev(src, dev, dtype), n, d0, s0, ny, dstride, sstride)
    check_equal("blit", to_np(d), O.blit(dst0.copy(), src, n, d0, s0, ny, dstride, sstride))


def test_blit_rejects_bad_arguments(qt, dev):
    a, b = torch.zeros(16, device=dev), torch.zeros(16, device=dev)
    with pytest.raises(ValueError):
        qt.batch.blit(a, b, 8, 12, 0)                                          # leaves the destination
    with pytest.raises(ValueError):
        qt.batch.blit(a, b, 8, 0, 4, ny=2, sstride=8)                          # leaves the source
    with pytest.raises(TypeError):
        qt.batch.blit(a, b.bfloat16(), 8, 0, 0)


def _small_cfg(qt):
    return qt.model.Cfg()


def test_pools_load_read_round_trip_and_neighbours(qt, dev):
    """Pools.load then Pools.read returns the state bit for bit; other slots, the other conv buffer and K / V rows >= pos keep
    their contents (reference tests/batch.py:59-71 checks the same properties on the decode step)"""
    cfg = _small_cfg(qt)
    S, Lmax, Lsrc, pos, slot = 3, 96, 64, 37, 1
    P = qt.batch.Pools(cfg, S, Lmax, device=dev)
    g = torch.Generator().manual_seed(5)
    for group in (P.conv, P.ssm, P.K, P.V):                                    # fill the pools so that stray writes would show
        for t in group:
            t.copy_(torch.randn(t.shape, generator=g).to(t.dtype))
    before = {k: [t.clone() for t in v] for k, v in P.as_tree().items()}
    nl, na = len(P.conv), len(P.K)
    state = {"conv": [torch.randn((1, 3, CD), generator=g).to(BF16).to(dev) for _ in range(nl)],
             "ssm": [torch.randn((1, HV, DV, DK), generator=g).to(dev) for _ in range(nl)],
             "kv": [(torch.randn((1, cfg.n_kv, Lsrc, cfg.head_dim), generator=g).to(BF16).to(dev),
                     torch.randn((1, cfg.n_kv, Lsrc, cfg.head_dim), generator=g).to(BF16).to(dev)) for _ in range(na)]}
    P.load(slot, state, pos)
    back = P.read(slot, pos, max_len=Lsrc)
    for i in range(nl):
        check_tensors_equal(f"conv {i}", back["conv"][i], state["conv"][i])
        check_tensors_equal(f"ssm {i}", back["ssm"][i], state["ssm"][i])
        check_tensors_equal(f"conv {i}: other parity buffer", P.conv[i][slot * 2 + ((pos & 1) ^ 1)], before["conv"][i][slot * 2 + ((pos & 1) ^ 1)])
        for other in (0, 2, 3):
            check_tensors_equal(f"ssm {i}: slot {other}", P.ssm[i][other], before["ssm"][i][other])
            check_tensors_equal(f"conv {i}: slot {other}", P.conv[i][other * 2:other * 2 + 2], before["conv"][i][other * 2:other * 2 + 2])
    for i in range(na):
        for name, pool, src, old in (("K", P.K[i], state["kv"][i][0], before["K"][i]), ("V", P.V[i], state["kv"][i][1], before["V"][i])):
            check_tensors_equal(f"{name} {i}: rows < pos", pool[slot, :, :pos], src[0, :, :pos])
            check_tensors_equal(f"{name} {i}: rows >= pos", pool[slot, :, pos:], old[slot, :, pos:])
            check_tensors_equal(f"{name} {i}: slot 0", pool[0], old[0])
        check_tensors_equal(f"read K {i}", back["kv"][i][0][0, :, :pos], state["kv"][i][0][0, :, :pos])
        if int(back["kv"][i][0][0, :, pos:].abs().sum().item()) != 0:
            raise AssertionError("read: rows past pos must be zero padding")


def test_plain_to_spec_to_plain_round_trip(qt, dev):
    """qwen35/serve.py:310-348: a sequence's recurrent state moves into snapshot 0 / conv buffer 0 of a snapshot-pool entry and,
    after a round that accepted n tokens, back from snapshot n; both moves are exact copies of the right buffers"""
    cfg = _small_cfg(qt)
    S, NS, M, Lmax = 3, 2, 4, 32
    P = qt.batch.Pools(cfg, S, Lmax, device=dev)
    SP = qt.batch_spec.SpecPools(cfg, NS, S, M, Lmax, device=dev)
    g = torch.Generator().manual_seed(6)
    for group in (P.conv, P.ssm, SP.conv, SP.ssm):
        for t in group:
            t.copy_(torch.randn(t.shape, generator=g).to(t.dtype))
    slot, pos, ss = 2, 11, 1
    want_conv = [c[slot * 2 + (pos & 1)].clone() for c in P.conv]
    want_ssm = [s[slot].clone() for s in P.ssm]
    sp_before = [s.clone() for s in SP.ssm]
    qt.batch_spec.to_spec(P, SP, slot, pos, ss)
    for i in range(len(P.conv)):
        check_tensors_equal(f"spec conv {i}", SP.conv[i][ss * 2, 0], want_conv[i])
        check_tensors_equal(f"spec ssm {i}", SP.ssm[i][ss, 0], want_ssm[i])
        check_tensors_equal(f"spec ssm {i}: other snapshots", SP.ssm[i][ss, 1:], sp_before[i][ss, 1:])
        check_tensors_equal(f"spec ssm {i}: other entries", SP.ssm[i][0], sp_before[i][0])
    # a round wrote snapshots 0..M-1 of buffer par = 1; n = 2 tokens were accepted: snapshot 2 is the live state at pos + 3
    par, n, new_pos = 1, 2, pos + 3
    live_conv = [c[(ss * 2 + par), n].clone() for c in SP.conv]
    live_ssm = [s[ss, n].clone() for s in SP.ssm]
    qt.batch_spec.to_plain(P, SP, slot, new_pos, ss, par, n)
    for i in range(len(P.conv)):
        check_tensors_equal(f"plain conv {i}", P.conv[i][slot * 2 + (new_pos & 1)], live_conv[i])
        check_tensors_equal(f"plain ssm {i}", P.ssm[i][slot], live_ssm[i])


def test_blit_batch_equals_single_blits(qt, dev):
    rng = np.random.default_rng(3)
    jobs, want = [], []
    for k, (n, d0, s0, ny, ds, ss, dt) in enumerate([(1024, 8, 16, 1, 0, 0, torch.float32), (18432, 36864, 0, 1, 0, 0, BF16),
                                                     (37 * 256, 96 * 256 * 2, 0, 2, 96 * 256, 64 * 256, BF16), (8, 0, 8, 5, 64, 16, BF16),
                                                     (262144, 262144, 0, 1, 0, 0, torch.float32)] * 14):          # 70 jobs: two launches
        nd, ns = d0 + (ny - 1) * ds + n + 16, s0 + (ny - 1) * ss + n + 8
        dst0, src = bf(rng.standard_normal(nd)), bf(rng.standard_normal(ns))
        d = to_dev(dst0, dev, dt)
        jobs.append((d, to_dev(src, dev, dt), n, d0, s0, ny, ds, ss))
        want.append(O.blit(dst0.copy(), src, n, d0, s0, ny, ds, ss))
    qt.batch.blit_batch(jobs)
    for k, (j, w) in enumerate(zip(jobs, want)):
        check_equal(f"job {k}", to_np(j[0]), w)
    with pytest.raises(ValueError):
        qt.batch.blit_batch([(jobs[0][0], jobs[0][1], 7, 0, 0, 1, 0, 0)])       # 28 bytes: not 16-byte granular


def test_blit_batch_with_empty_jobs_and_more_units_than_workgroups(qt, dev):
    """A launch is one flat space of 16 KiB units over all its copies.  Here: copies of no rows or no elements before, between and
    behind the others (their unit ranges are empty), rows that end inside a unit, and one copy of 48 MiB, which gives every
    workgroup several units with the next one requested before the current one is stored."""
    rng = np.random.default_rng(4)
    shapes = [(0, 0, 0, 3, 16, 16, BF16), (4096 + 8, 8, 0, 3, 8192, 4104, BF16), (128, 0, 0, 0, 0, 0, torch.float32),
              (12 << 20, 4, 8, 1, 0, 0, torch.float32), (0, 0, 0, 1, 0, 0, BF16), (8, 8, 0, 7, 16, 8, BF16), (16, 0, 0, 0, 0, 0, BF16)]
    jobs, want = [], []
    for n, d0, s0, ny, ds, ss, dt in shapes:
        nd, ns = d0 + max(ny - 1, 0) * ds + n + 16, s0 + max(ny - 1, 0) * ss + n + 8
        dst0 = bf(rng.standard_normal(nd))
        src = bf(rng.standard_normal(ns))
        jobs.append((to_dev(dst0, dev, dt), to_dev(src, dev, dt), n, d0, s0, ny, ds, ss))
        want.append(O.blit(dst0.copy(), src, n, d0, s0, ny, ds, ss) if n and ny else dst0)
    qt.batch.blit_batch(jobs)
    for k, (j, w) in enumerate(zip(jobs, want)):
        check_equal(f"job {k}", to_np(j[0]), w)
    qt.batch.blit_batch([jobs[0], jobs[2]])                                  # nothing to move at all
    check_equal("empty launch", to_np(jobs[0][0]), want[0])
