"""GPU parity of the ragged GQA hd256 decode / verify attention against the CPU oracle (float64 softmax attention).
Tolerance (the stated target): bf16 attention outputs within 1e-2 relative."""
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


def check_attn(name, got, ref):
    check_rel(name + " rel-L2", got, ref, 1e-2, rel_l2)
    check_rel(name + " max", got, ref, 1e-2, rel_max)


def run_case(qt, dev, rng, S, Lmax, slots, pos, M, split=None):
    B = len(slots)
    Kp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    Vp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    q = bf(rng.standard_normal((B * M, 8, 256)))
    kn = bf(rng.standard_normal((B * M, 2, 256)))
    vn = bf(rng.standard_normal((B * M, 2, 256)))
    dK, dV = to_dev(Kp, dev, BF16), to_dev(Vp, dev, BF16)
    o = qt.batch.attn_b(to_dev(q, dev, BF16), to_dev(kn, dev, BF16), to_dev(vn, dev, BF16), dK, dV, to_dev(slots, dev), to_dev(pos, dev),
                        M, split=split)
    oK, oV = Kp.copy(), Vp.copy()
    ref = O.attn_b(q, kn, vn, oK, oV, slots, pos, M)
    got = to_np(o)
    for r in range(B * M):                                                     # per query row: a short row's large outputs must not
        check_attn(f"o row {r} (sequence {r // M}, M={M})", got[r], ref[r])    # hide a long row's small ones
    check_equal("K pool (appended rows, everything else untouched)", to_np(dK), oK)
    check_equal("V pool", to_np(dV), oV)
    return to_np(o)


def test_attn_b_layout_of_reference_test(qt, dev):
    """reference tests/batch.py:73-100: 6 rows, positions 0..1023, slots scattered in a 7-slot pool"""
    rng = np.random.default_rng(11)
    run_case(qt, dev, rng, 6, 1024, np.array([3, 0, 5, 1, 2, 4], np.int32), np.array([0, 1, 31, 32, 300, 1023], np.int32), 1)


@pytest.mark.parametrize("M", [2, 3, 4, 5, 6, 8, 9, 16])
def test_attn_b_verify_rows(qt, dev, M):
    """reference tests/batch_spec.py:69-101: M query rows per sequence, causal among the new keys"""
    rng = np.random.default_rng(M)
    run_case(qt, dev, rng, 6, 1024, np.array([3, 0, 5, 1, 2], np.int32), np.array([0, 1, 30, 300, 1000], np.int32), M)


def test_attn_b_split_invariance_and_single_key(qt, dev):
    rng = np.random.default_rng(5)
    slots, pos = np.array([1, 0], np.int32), np.array([777, 0], np.int32)
    outs = []
    for split in (16, 64, 256, 1024):
        rng2 = np.random.default_rng(5)
        outs.append(run_case(qt, dev, rng2, 2, 1024, slots, pos, 1, split=split))
    for o in outs[1:]:
        check_rel("split count changes the result only by rounding", o, outs[0], 1e-2, rel_max)
    # a sequence at position 0 sees exactly one key (its own): o = v for every head of the group
    rng3 = np.random.default_rng(5)
    Kp = bf(rng3.standard_normal((3, 2, 1024, 256)))
    Vp = bf(rng3.standard_normal((3, 2, 1024, 256)))
    q = bf(rng3.standard_normal((2, 8, 256)))
    kn = bf(rng3.standard_normal((2, 2, 256)))
    vn = bf(rng3.standard_normal((2, 2, 256)))
    check_equal("single key: o == v", outs[0][1], np.repeat(vn[1], 4, axis=0))


def test_attn_b_out_of_range_rows_are_skipped(qt, dev):
    rng = np.random.default_rng(6)
    Kp = to_dev(bf(rng.standard_normal((3, 2, 64, 256))), dev, BF16)
    Vp = to_dev(bf(rng.standard_normal((3, 2, 64, 256))), dev, BF16)
    K0, V0 = Kp.clone(), Vp.clone()
    q = to_dev(bf(rng.standard_normal((2, 8, 256))), dev, BF16)
    kn = to_dev(bf(rng.standard_normal((2, 2, 256))), dev, BF16)
    qt.batch.attn_b(q, kn, kn, Kp, Vp, torch.tensor([5, 1], dtype=torch.int32, device=dev), torch.tensor([3, 64], dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    check_tensors_equal("pools untouched by a bad slot / a full sequence", Kp, K0)
    check_tensors_equal("pools untouched", Vp, V0)
    with pytest.raises(ValueError):
        qt.batch.attn_b(q, kn, kn, Kp, Vp, torch.tensor([0], dtype=torch.int32, device=dev), torch.tensor([0], dtype=torch.int32, device=dev), M=17)


@pytest.mark.parametrize("M", [5, 8])
def test_attn_b_more_than_four_tokens_full_or_bad_rows(qt, dev, M):
    """the reference kernel is generic in M (qwen35/batch.py:230-237, run.py:15 lets k be anything): a sequence whose M rows do
    not all fit, or whose slot is outside the pool, is skipped as a whole by every pass (nothing of it is appended); its
    neighbours are computed, rows of the later passes included"""
    rng = np.random.default_rng(70 + M)
    Lmax, S = 96, 4
    slots = np.array([2, 9, 0, 1], np.int32)                                   # slot 9 is outside the pool
    pos = np.array([Lmax - M, 5, Lmax - M + 1, 0], np.int32)                    # sequence 2: one row too many
    Kp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    Vp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    q = bf(rng.standard_normal((4 * M, 8, 256)))
    kn = bf(rng.standard_normal((4 * M, 2, 256)))
    vn = bf(rng.standard_normal((4 * M, 2, 256)))
    dK, dV = to_dev(Kp, dev, BF16), to_dev(Vp, dev, BF16)
    o = to_np(qt.batch.attn_b(to_dev(q, dev, BF16), to_dev(kn, dev, BF16), to_dev(vn, dev, BF16), dK, dV, to_dev(slots, dev),
                              to_dev(pos, dev), M))
    oK, oV = Kp.copy(), Vp.copy()
    good = np.array([0, 3])
    rows = (good[:, None] * M + np.arange(M)[None]).ravel()
    ref = O.attn_b(q[rows], kn[rows], vn[rows], oK, oV, slots[good], pos[good], M)
    for i, r in enumerate(rows):
        check_attn(f"o row {r}", o[r], ref[i])
    check_equal("K pool", to_np(dK), oK)
    check_equal("V pool", to_np(dV), oV)


@pytest.mark.parametrize("B,M,Lmax", [(64, 1, 640), (64, 4, 640), (40, 1, 640), (40, 3, 640), (130, 2, 640), (300, 4, 200),
                                      (1024, 1, 96)])
def test_attn_b_many_sequences(qt, dev, B, M, Lmax):
    """more (sequence, KV head) segments than one 64-lane scan step of the segment table holds (B > 32), many segments per
    workgroup, and more segments than workgroups' worth of tiles, up to the 1024 sequences (2048 segments) the entry point
    takes: ragged positions including 0, 1 and the last position that fits, a few rows with an out-of-range slot or a full
    sequence (skipped: their outputs are not defined and not compared), every other row against the oracle row by row, the
    pools bit-exact outside the appended rows"""
    rng = np.random.default_rng(100 * B + M)
    S = B + 3
    slots = rng.permutation(S)[:B].astype(np.int32)
    pos = rng.integers(0, Lmax - M, B).astype(np.int32)
    pos[:6] = [0, 1, Lmax - M, 15, 16, 17]
    pos[B // 2:B // 2 + 8] = rng.integers(0, 40, 8)                             # a run of very short sequences: many segments in one workgroup
    bad = np.zeros(B, bool)
    slots[7], bad[7] = S + 5, True                                              # slot outside the pool
    slots[B - 2], bad[B - 2] = -1, True
    pos[9], bad[9] = Lmax - M + 1, True                                         # the M rows would not fit
    Kp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    Vp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    q = bf(rng.standard_normal((B * M, 8, 256)))
    kn = bf(rng.standard_normal((B * M, 2, 256)))
    vn = bf(rng.standard_normal((B * M, 2, 256)))
    dK, dV = to_dev(Kp, dev, BF16), to_dev(Vp, dev, BF16)
    o = to_np(qt.batch.attn_b(to_dev(q, dev, BF16), to_dev(kn, dev, BF16), to_dev(vn, dev, BF16), dK, dV, to_dev(slots, dev),
                              to_dev(pos, dev), M))
    oK, oV = Kp.copy(), Vp.copy()
    good = np.flatnonzero(~bad)
    rows = (good[:, None] * M + np.arange(M)[None]).ravel()
    ref = O.attn_b(q[rows], kn[rows], vn[rows], oK, oV, slots[good], pos[good], M)
    for i, r in enumerate(rows):
        check_attn(f"row {r} (sequence {r // M}, pos {pos[r // M]})", o[r], ref[i])
    check_equal("K pool (appended rows, everything else untouched)", to_np(dK), oK)
    check_equal("V pool", to_np(dV), oV)


def test_attn_b_config3_ragged_long(qt, dev):
    """benchmark config 3: B=16, one query each, ragged KV lengths uniform in [512, 32768] (seed 1003)"""
    rng = np.random.default_rng(1003)
    B, Lmax = 16, 32768
    pos = rng.integers(512, 32768, B).astype(np.int32)                          # keys already in the pool (+1 new)
    pos[0], pos[1] = 32767, 512
    slots = rng.permutation(B).astype(np.int32)
    g = torch.Generator().manual_seed(1003)
    Kp = torch.randn((B + 1, 2, Lmax, 256), generator=g, dtype=torch.float32).bfloat16()
    Vp = torch.randn((B + 1, 2, Lmax, 256), generator=g, dtype=torch.float32).bfloat16()
    q = bf(rng.standard_normal((B, 8, 256)))
    kn = bf(rng.standard_normal((B, 2, 256)))
    vn = bf(rng.standard_normal((B, 2, 256)))
    dK, dV = Kp.to(dev), Vp.to(dev)
    o = to_np(qt.batch.attn_b(to_dev(q, dev, BF16), to_dev(kn, dev, BF16), to_dev(vn, dev, BF16), dK, dV, to_dev(slots, dev), to_dev(pos, dev)))
    for b in range(B):                                                         # oracle per sequence on views (no 2 GB copies)
        s_, p = int(slots[b]), int(pos[b])
        Kb = Kp[s_:s_ + 1, :, :p + 1].float().numpy().copy()
        Vb = Vp[s_:s_ + 1, :, :p + 1].float().numpy().copy()
        ref = O.attn_b(q[b:b + 1], kn[b:b + 1], vn[b:b + 1], Kb, Vb, np.array([0]), np.array([p]), 1)
        check_attn(f"sequence {b} (L={p + 1})", o[b:b + 1], ref)
        check_equal("appended K row", to_np(dK[s_, :, p]), kn[b])
        check_equal("appended V row", to_np(dV[s_, :, p]), vn[b])
    check_tensors_equal("trash slot untouched", dK[B].cpu(), Kp[B])


def test_attn_b_config4_verify_mix(qt, dev):
    """benchmark config 4 (attention half): B=16 x M=4, KV lengths uniform in [1024, 8192], 4-token causal tail"""
    rng = np.random.default_rng(1004)
    B, M, Lmax = 16, 4, 8192 + 8
    pos = rng.integers(1024, 8192, B).astype(np.int32)
    slots = rng.permutation(B).astype(np.int32)
    run_case(qt, dev, rng, B, Lmax, slots, pos, M)


# ------------------------------------------------------------------------------------- causal prefill attention
@pytest.mark.parametrize("S,L", [(1, 1), (5, 5), (64, 64), (100, 100), (37, 200), (300, 300), (128, 1000),
                                 (63, 63), (65, 65), (129, 129), (1, 64), (2, 65), (70, 135), (64, 128), (17, 1025)])
def test_prefill_causal_vs_oracle(qt, dev, S, L):
    """softmax(Q K^T / 16 + causal) V, GQA 8/2, D=256 (model.py:160-167); with L > S the queries are the last S positions"""
    rng = np.random.default_rng(S * 1000 + L)
    q = bf(rng.standard_normal((8, S, 256)))
    K = bf(rng.standard_normal((2, L + 7, 256)))
    V = bf(rng.standard_normal((2, L + 7, 256)))
    dK, dV = to_dev(K, dev, BF16)[None], to_dev(V, dev, BF16)[None]
    o = qt.attention.scaled_dot_product_attention(to_dev(q, dev, BF16)[None], dK[:, :, :L], dV[:, :, :L], scale=256 ** -0.5, mask="causal")
    ref = O.sdpa_causal(q, K[:, :L], V[:, :L])
    check_attn(f"S={S} L={L}", to_np(o)[0], ref)


def test_prefill_causal_2048(qt, dev):
    rng = np.random.default_rng(2048)
    S = 2048
    q = bf(rng.standard_normal((8, S, 256)))
    K = bf(rng.standard_normal((2, S, 256)))
    V = bf(rng.standard_normal((2, S, 256)))
    o = to_np(qt.attention.scaled_dot_product_attention(to_dev(q, dev, BF16)[None], to_dev(K, dev, BF16)[None], to_dev(V, dev, BF16)[None],
                                                        scale=256 ** -0.5, mask="causal"))[0]
    ref = O.sdpa_causal(q, K, V)
    check_attn("S=2048", o, ref)
    # the first row sees one key: o = v
    check_equal("row 0 == v[0]", o[:, 0], np.repeat(V[:, 0], 4, axis=0))
    with pytest.raises(ValueError):
        qt.attention.scaled_dot_product_attention(to_dev(q, dev, BF16)[None], to_dev(K, dev, BF16)[None], to_dev(V, dev, BF16)[None],
                                                  scale=256 ** -0.5, mask=None)


def test_prefill_causal_8192_two_heads_per_wavefront(qt, dev):
    """S = 8192 (the long-prefill benchmark size; the launch uses 32-row workgroups with two heads per wavefront): a sample of query
    rows, including block borders and the first / last rows, against the float64 oracle evaluated for those rows only"""
    rng = np.random.default_rng(8192)
    S = 8192
    g = torch.Generator().manual_seed(8192)
    q = torch.randn((8, S, 256), generator=g).bfloat16()
    K = torch.randn((2, S, 256), generator=g).bfloat16()
    V = torch.randn((2, S, 256), generator=g).bfloat16()
    o = to_np(qt.attention.scaled_dot_product_attention(q.to(dev)[None], K.to(dev)[None], V.to(dev)[None], scale=256 ** -0.5,
                                                        mask="causal"))[0]
    rows = sorted(set([0, 1, 15, 16, 31, 32, 33, 63, 64, 65, 4095, 4096, 8159, 8160, 8176, 8191] + [int(r) for r in rng.integers(0, S, 40)]))
    qn, Kn, Vn = q.float().numpy(), K.float().numpy(), V.float().numpy()
    for r in rows:
        ref = O.sdpa_causal(qn[:, r:r + 1], Kn[:, :r + 1], Vn[:, :r + 1])            # the row at position r sees keys 0..r
        check_attn(f"S=8192 row {r}", o[:, r:r + 1], ref)
    check_equal("row 0 == v[0]", o[:, 0], np.repeat(Vn[:, 0], 4, axis=0))


@pytest.mark.parametrize("S", [2048, 4800])
def test_prefill_causal_reference_points_that_move_late(qt, dev, S):
    """Two heads per wavefront, split along the keys (S = 2048) and unsplit (S = 4800).  The kernel exponentiates a tile against the
    running reference points before it knows the tile's maxima and takes the tile again when a row's maximum grew by more
    than 2^8: here a handful of keys deep inside the sequence are aligned with a block of query rows and scaled up, so that rows
    which have settled long ago jump by 2^14 .. 2^187 in one tile (the last ones overflow the exponential taken on the bet), some
    rows of a wavefront and not others, more than once."""
    g = torch.Generator().manual_seed(S)
    q = torch.randn((8, S, 256), generator=g)
    K = torch.randn((2, S, 256), generator=g)
    V = torch.randn((2, S, 256), generator=g).bfloat16()
    rng = np.random.default_rng(S)
    special = sorted(int(k) for k in rng.choice(np.arange(300, S - 200), 6, replace=False))
    for j, k in enumerate(special):
        h = int(rng.integers(0, 8))
        r0 = k + int(rng.integers(1, 150))                       # rows that see the key: a ragged set across wavefront borders
        rows = slice(r0, min(S, r0 + int(rng.integers(3, 40))))
        K[h // 4, k] = q[h, r0] * (0.6 + 1.5 * j)                # score ~ |q|^2 (0.6 .. 8.1) / 16 = 10 .. 130 (base e) above the rest
        q[h, rows] = q[h, r0] + 0.05 * torch.randn((rows.stop - rows.start, 256), generator=g)
    q, K = q.bfloat16(), K.bfloat16()
    o = to_np(qt.attention.scaled_dot_product_attention(q.to(dev)[None], K.to(dev)[None], V.to(dev)[None], scale=256 ** -0.5,
                                                        mask="causal"))[0]
    qn, Kn, Vn = q.float().numpy(), K.float().numpy(), V.float().numpy()
    rows = set(int(r) for r in rng.integers(0, S, 24))
    for k in special:
        rows.update(range(k - 2, min(S, k + 190), 7))
    for r in sorted(rows):
        check_attn(f"S={S} row {r}", o[:, r:r + 1], O.sdpa_causal(qn[:, r:r + 1], Kn[:, :r + 1], Vn[:, :r + 1]))


@pytest.mark.parametrize("S,P0", [(4800, 0), (2048, 0), (1536, 1000), (6001, 333)])
def test_prefill_causal_two_role_kernel_is_repeatable(qt, dev, S, P0):
    """From about 1500 rows on, a workgroup's wavefronts work in pairs: one computes a tile's scores and softmax and hands P (with
    the rows' rescale factors) to its partner through LDS, one tile ahead of the partner's P.V.  An access of that hand-over that
    is not ordered shows as a result that depends on timing: five calls on the same inputs (unsplit, split, after a prefix,
    ragged) must agree in every bit, with other work on the GPU between them."""
    L = S + P0
    g = torch.Generator().manual_seed(S + P0)
    q = torch.randn((1, 8, S, 256), generator=g).bfloat16().to(dev)
    K = torch.randn((1, 2, L, 256), generator=g).bfloat16().to(dev)
    V = torch.randn((1, 2, L, 256), generator=g).bfloat16().to(dev)
    first = qt.attention.scaled_dot_product_attention(q, K, V, scale=256 ** -0.5, mask="causal").clone()
    assert bool(torch.isfinite(first.float()).all())
    for i in range(4):
        (K.float() * (i + 2)).sum().item()                       # unrelated kernels and a synchronisation in between
        again = qt.attention.scaled_dot_product_attention(q, K, V, scale=256 ** -0.5, mask="causal")
        assert torch.equal(first, again), f"call {i + 2} differs from the first"


def test_prefill_causal_long_ragged_continuation(qt, dev):
    """two heads per wavefront with nothing aligned: S = 8170 query rows continue a prefix of 37 keys (L = 8207: the last tile is
    shifted back, the last row blocks are partial, some wavefronts have one tile less than their workgroup)"""
    rng = np.random.default_rng(8170)
    S, P0 = 8170, 37
    L = S + P0
    g = torch.Generator().manual_seed(8170)
    q = torch.randn((8, S, 256), generator=g).bfloat16()
    K = torch.randn((2, L, 256), generator=g).bfloat16()
    V = torch.randn((2, L, 256), generator=g).bfloat16()
    o = to_np(qt.attention.scaled_dot_product_attention(q.to(dev)[None], K.to(dev)[None], V.to(dev)[None], scale=256 ** -0.5,
                                                        mask="causal"))[0]
    rows = sorted(set([0, 1, 15, 16, 26, 27, 31, 32, 8127, 8128, 8159, 8160, 8161, 8168, 8169] + [int(r) for r in rng.integers(0, S, 30)]))
    qn, Kn, Vn = q.float().numpy(), K.float().numpy(), V.float().numpy()
    for r in rows:
        ref = O.sdpa_causal(qn[:, r:r + 1], Kn[:, :P0 + r + 1], Vn[:, :P0 + r + 1])   # the row at position P0 + r sees keys 0..P0 + r
        check_attn(f"continuation row {r}", o[:, r:r + 1], ref)


@pytest.mark.parametrize("qscale", [0.05, 6.0, 40.0])
def test_prefill_causal_score_ranges(qt, dev, qscale):
    """flat scores (no row is ever rescaled after the first tile), scores whose maxima keep jumping by more than the rescale
    threshold, and near one-hot softmax rows"""
    rng = np.random.default_rng(int(qscale * 100))
    S = 400
    q = bf(rng.standard_normal((8, S, 256)) * qscale)
    K = bf(rng.standard_normal((2, S, 256)))
    V = bf(rng.standard_normal((2, S, 256)))
    o = qt.attention.scaled_dot_product_attention(to_dev(q, dev, BF16)[None], to_dev(K, dev, BF16)[None], to_dev(V, dev, BF16)[None],
                                                  scale=256 ** -0.5, mask="causal")
    check_attn(f"q scale {qscale}", to_np(o)[0], O.sdpa_causal(q, K, V))


@pytest.mark.parametrize("S,P0,qscale", [(1024, 0, 1.0), (1000, 23, 1.0), (100, 1007, 1.0), (64, 8000, 1.0), (300, 4001, 1.0),
                                         (1024, 3000, 1.0), (16, 5000, 1.0), (1, 4095, 1.0), (1000, 9, 40.0), (130, 2000, 0.05),
                                         # from about 1500 rows on: 32-row blocks, two heads per wavefront, with the split
                                         (1536, 0, 1.0), (2048, 0, 1.0), (1500, 23, 1.0), (2500, 7, 40.0), (1800, 5000, 1.0),
                                         (2816, 0, 0.05), (3200, 0, 1.0), (2049, 2048, 1.0)])
def test_prefill_causal_key_split(qt, dev, S, P0, qscale):
    """Launches that leave half of the CUs idle are split along the keys (parts of a row block meet in a workspace and a second
    kernel combines them): prompts of up to 3200 rows and continuations of a long prefix, positions that are no
    multiple of 16 (some rows of a block then see no key of the block's last part), rescaled and flat score ranges.  Checked
    against the float64 oracle on a sample of rows, and against the same launch without a workspace (unsplit)."""
    from qwen_tailor_amd import _lib as QL
    rng = np.random.default_rng(S * 7 + P0)
    L = S + P0
    g = torch.Generator().manual_seed(S * 7 + P0)
    q = (torch.randn((8, S, 256), generator=g) * qscale).bfloat16()
    K = torch.randn((2, L, 256), generator=g).bfloat16()
    V = torch.randn((2, L, 256), generator=g).bfloat16()
    assert QL.lib().qt_gqa_prefill_workspace_bytes_for(S, L, P0) > 0, "this case is meant to be split"
    assert QL.lib().qt_gqa_prefill_workspace_bytes_for(S, L, P0) <= QL.lib().qt_gqa_prefill_workspace_bytes(L)
    dq, dK, dV = q.to(dev)[None], K.to(dev)[None], V.to(dev)[None]
    o = qt.attention.scaled_dot_product_attention(dq, dK, dV, scale=256 ** -0.5, mask="causal")
    plain = torch.full_like(o, float("nan"))
    QL.call("qt_gqa_prefill_causal", QL.ptr(dq), QL.ptr(dK), QL.ptr(dV), QL.ptr(plain), None, 0, S, L, P0, S * 256, L * 256, QL.stream())
    o, plain = to_np(o)[0], to_np(plain)[0]
    assert np.isfinite(o).all() and np.isfinite(plain).all()
    check_attn("split against unsplit", o, plain)
    rows = sorted(set([0, 1, 15, 16, 17, S // 2, S - 17, S - 16, S - 2, S - 1] + [int(r) for r in rng.integers(0, S, 24)]) & set(range(S)))
    qn, Kn, Vn = q.float().numpy(), K.float().numpy(), V.float().numpy()
    for r in rows:
        ref = O.sdpa_causal(qn[:, r:r + 1], Kn[:, :P0 + r + 1], Vn[:, :P0 + r + 1])
        check_attn(f"S={S} P0={P0} row {r}", o[:, r:r + 1], ref)


@pytest.mark.parametrize("S,P0", [(1024, 0), (2048, 0), (300, 3000), (5000, 0)])
def test_prefill_causal_head_strides(qt, dev, S, P0):
    """q / out with a head stride beyond S rows and K / V inside a longer cache, through the C ABI, in every form of the launch
    (16- and 32-row blocks, split and unsplit): same bits as the contiguous call, and nothing written between the heads"""
    from qwen_tailor_amd import _lib as QL
    L, pad = S + P0, 5
    g = torch.Generator().manual_seed(S + P0)
    q = torch.randn((8, S, 256), generator=g).bfloat16().to(dev)
    K = torch.randn((2, L + 9, 256), generator=g).bfloat16().to(dev)
    V = torch.randn((2, L + 9, 256), generator=g).bfloat16().to(dev)
    want = qt.attention.scaled_dot_product_attention(q[None], K[None, :, :L], V[None, :, :L], scale=256 ** -0.5, mask="causal")[0]
    qs = torch.zeros((8, S + pad, 256), dtype=BF16, device=dev)
    qs[:, :S] = q
    outs = torch.full((8, S + pad, 256), 7.0, dtype=BF16, device=dev)
    nws = QL.lib().qt_gqa_prefill_workspace_bytes_for(S, L, P0)
    ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dev)
    QL.call("qt_gqa_prefill_causal", QL.ptr(qs), QL.ptr(K), QL.ptr(V), QL.ptr(outs), QL.ptr(ws), nws, S, L, P0, (S + pad) * 256, (L + 9) * 256,
            QL.stream())
    assert torch.equal(outs[:, :S], want), "strided call differs from the contiguous one"
    assert bool((outs[:, S:] == 7.0).all()), "rows between the heads were written"


def test_prefill_causal_split_equals_unsplit_on_random_shapes(qt, dev):
    """Forty launches of random size and prefix, each run with the workspace its split asks for and without one (unsplit): the two
    agree to rounding, every output row is written, and the workspace need stays within the bound for its key count."""
    from qwen_tailor_amd import _lib as QL
    rng = np.random.default_rng(20240)
    g = torch.Generator().manual_seed(20240)
    nsplit = 0
    for case in range(40):
        S = int(rng.choice([rng.integers(1, 200), rng.integers(200, 1500), rng.integers(1500, 3000)]))
        P0 = int(rng.choice([0, rng.integers(1, 300), rng.integers(300, 9000)]))
        L = S + P0
        q = torch.randn((8, S, 256), generator=g).bfloat16().to(dev)
        K = torch.randn((2, L, 256), generator=g).bfloat16().to(dev)
        V = torch.randn((2, L, 256), generator=g).bfloat16().to(dev)
        nws = QL.lib().qt_gqa_prefill_workspace_bytes_for(S, L, P0)
        assert 0 <= nws <= QL.lib().qt_gqa_prefill_workspace_bytes(L), (S, P0, nws)
        nsplit += nws > 0
        outs = []
        for ws_bytes in (nws, 0):
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
            out = torch.full((8, S, 256), float("nan"), dtype=BF16, device=dev)
            QL.call("qt_gqa_prefill_causal", QL.ptr(q), QL.ptr(K), QL.ptr(V), QL.ptr(out), QL.ptr(ws) if ws_bytes else None, ws_bytes,
                    S, L, P0, S * 256, L * 256, QL.stream())
            outs.append(to_np(out))
        assert np.isfinite(outs[0]).all() and np.isfinite(outs[1]).all(), (case, S, P0)
        check_attn(f"case {case}: S={S} P0={P0}", outs[0], outs[1])
    assert nsplit >= 10, nsplit                                   # the sample does exercise the split


def test_prefill_causal_rejects_queries_past_the_keys(qt, dev):
    from qwen_tailor_amd import _lib as QL
    t = torch.zeros((1, 8, 32, 256), dtype=BF16, device=dev)
    kv = torch.zeros((1, 2, 40, 256), dtype=BF16, device=dev)
    with pytest.raises(RuntimeError):
        QL.call("qt_gqa_prefill_causal", QL.ptr(t), QL.ptr(kv), QL.ptr(kv), QL.ptr(t), None, 0, 32, 40, 9, 32 * 256, 40 * 256, QL.stream())


# ------------------------------------------------------------------------------------- glue either side of the attention kernels
@pytest.mark.parametrize("R,M", [(1, 1), (5, 1), (8, 4), (64, 1), (259, 1), (2048, 4)])
def test_qkv_prep_and_out_gate_bit_exact(qt, dev, R, M):
    """q / k RMSNorm + partial RoPE + v split, and o * sigmoid(gate) (batch.py:505-513): every bf16 value equals the oracle's"""
    rng = np.random.default_rng(100 * R + M)
    qkv = bf(rng.standard_normal((R, O.QKV_W)) * 2)
    qn, kn = bf(1 + 0.2 * rng.standard_normal(256)), bf(1 + 0.2 * rng.standard_normal(256))
    pos = rng.integers(0, 32768, R // M).astype(np.int32)
    pos[0] = 0
    dq = to_dev(qkv, dev, BF16)
    q, k, v = qt.attention.qkv_prep(dq, to_dev(qn, dev, BF16), to_dev(kn, dev, BF16), to_dev(pos, dev), M)
    oq, ok, ov = O.attn_qkv_prep(qkv, qn, kn, pos, M)
    check_equal("q", to_np(q), oq)
    check_equal("k", to_np(k), ok)
    check_equal("v", to_np(v), ov)
    # the same with the rotary pairs read from the device's table: every position inside it, and a table that ends below
    # most positions (those rows evaluate their own pairs): the same bits either way
    for bound in (int(pos.max()) + M, 1000):
        qt_, kt_, vt_ = qt.attention.qkv_prep(dq, to_dev(qn, dev, BF16), to_dev(kn, dev, BF16), to_dev(pos, dev), M, max_pos=bound)
        assert torch.equal(qt_, q) and torch.equal(kt_, k) and torch.equal(vt_, v), f"table up to {bound}"
    o = bf(rng.standard_normal((R, 8, 256)))
    if R >= 256:                                                 # tiny, huge, zero and -0 gates among the ordinary ones
        special = bf(np.array([1e-7, -3e-6, 200.0, -150.0, 0.0, -0.0, 127.5, -1e-30]))
        for h in (0, 3, 6):
            blk = qkv[::7, h * 512 + 256:(h + 1) * 512:5]        # a view: every 5th gate of head h in every 7th row
            blk[...] = special[rng.integers(0, 8, blk.shape)]
        dq = to_dev(qkv, dev, BF16)
    check_equal("gated output", to_np(qt.attention.out_gate(to_dev(o, dev, BF16), dq)), O.attn_out_gate(o, qkv))


def test_attention_layer_core_decode_rows(qt, dev):
    """qkv_prep -> attn_b -> out_gate on 5 decode rows against the same chain of oracle functions (a full-attention layer between
    its qkv and o_proj projections, batch.py:504-514)"""
    rng = np.random.default_rng(77)
    B, Lmax = 5, 256
    slots, pos = np.array([3, 0, 4, 1, 2], np.int32), np.array([0, 1, 100, 255 - 1, 17], np.int32)
    qkv = bf(rng.standard_normal((B, O.QKV_W)))
    qn, kn = bf(1 + 0.1 * rng.standard_normal(256)), bf(1 + 0.1 * rng.standard_normal(256))
    Kp, Vp = bf(rng.standard_normal((6, 2, Lmax, 256))), bf(rng.standard_normal((6, 2, Lmax, 256)))
    dq, dK, dV = to_dev(qkv, dev, BF16), to_dev(Kp, dev, BF16), to_dev(Vp, dev, BF16)
    q, k, v = qt.attention.qkv_prep(dq, to_dev(qn, dev, BF16), to_dev(kn, dev, BF16), to_dev(pos, dev))
    o = qt.batch.attn_b(q, k, v, dK, dV, to_dev(slots, dev), to_dev(pos, dev))
    out = qt.attention.out_gate(o, dq)
    oq, ok, ov = O.attn_qkv_prep(qkv, qn, kn, pos)
    oo = O.attn_b(oq, ok, ov, Kp, Vp, slots, pos, 1)
    check_rel("layer core", to_np(out), O.attn_out_gate(oo, qkv), 1e-2, rel_max)
    check_equal("appended K", to_np(dK), Kp)                                   # the oracle appended the same rows in place


def _layer_case(qt, dev, seed, B, M, Lmax, lo, hi, bad=False):
    """the three-call chain (qkv_prep, attn_b, out_gate) and the two-launch layer form on the same inputs; returns both results"""
    rng = np.random.default_rng(seed)
    S = B + 2
    slots = rng.permutation(S)[:B].astype(np.int32)
    pos = rng.integers(lo, hi, B).astype(np.int32)
    pos[0] = lo
    if bad:
        slots[1], pos[B - 1] = S + 3, Lmax - M + 1                              # skipped rows: outputs undefined, pools untouched
    qkv = bf(rng.standard_normal((B * M, O.QKV_W)) * 1.5)
    qn, kn = bf(1 + 0.2 * rng.standard_normal(256)), bf(1 + 0.2 * rng.standard_normal(256))
    Kp = to_dev(bf(rng.standard_normal((S + 1, 2, Lmax, 256))), dev, BF16)
    Vp = to_dev(bf(rng.standard_normal((S + 1, 2, Lmax, 256))), dev, BF16)
    dq, dqn, dkn, dslots, dpos = to_dev(qkv, dev, BF16), to_dev(qn, dev, BF16), to_dev(kn, dev, BF16), to_dev(slots, dev), to_dev(pos, dev)
    K1, V1 = Kp.clone(), Vp.clone()
    q, k, v = qt.attention.qkv_prep(dq, dqn, dkn, dpos, M)
    want = qt.attention.out_gate(qt.batch.attn_b(q, k, v, K1, V1, dslots, dpos, M), dq)
    K2, V2 = Kp.clone(), Vp.clone()
    got = qt.batch.attn_layer_b(dq, dqn, dkn, K2, V2, dslots, dpos, M)
    good = np.ones(B, bool)
    if bad:
        good[[1, B - 1]] = False
    rows = torch.from_numpy(np.flatnonzero(np.repeat(good, M))).to(dev)
    check_tensors_equal(f"layer form, outputs (B={B}, M={M})", got[rows], want[rows])
    check_tensors_equal("layer form, K pool", K2, K1)
    check_tensors_equal("layer form, V pool", V2, V1)
    return qkv, qn, kn, slots, pos, to_np(Kp), to_np(Vp), to_np(got), good


@pytest.mark.parametrize("B,M,Lmax,lo,hi", [(5, 1, 256, 0, 250), (6, 4, 1024, 0, 1000), (3, 2, 96, 0, 90), (16, 3, 640, 0, 600),
                                            (40, 1, 640, 0, 630), (130, 2, 200, 0, 190), (4, 7, 300, 0, 290), (2, 16, 128, 0, 100)])
def test_attention_layer_two_launches_equal_the_three_calls(qt, dev, B, M, Lmax, lo, hi):
    """batch.attn_layer_b (q / k norm and rotary embedding inside the attention kernel, the output gate in the merge) against
    attention.qkv_prep -> batch.attn_b -> attention.out_gate: the same bits in the outputs and in the pools, also with skipped
    rows, with more segments than workgroups and with more than four tokens per sequence; and against the oracle chain"""
    qkv, qn, kn, slots, pos, Kp, Vp, got, good = _layer_case(qt, dev, 500 + B + M, B, M, Lmax, lo, hi, bad=B >= 5)
    if B * M <= 64:
        keep = np.flatnonzero(good)
        rows = (keep[:, None] * M + np.arange(M)[None]).ravel()
        oq, ok, ov = O.attn_qkv_prep(qkv[rows], qn, kn, pos[keep], M)
        oo = O.attn_b(oq, ok, ov, Kp, Vp, slots[keep], pos[keep], M)
        ref = O.attn_out_gate(oo, qkv[rows])
        for i, r in enumerate(rows):
            check_attn(f"row {r} against the oracle chain", got[r], ref[i])


def test_attention_layer_config4_two_launches(qt, dev):
    """benchmark config 4's attention half (B = 16 x M = 4, ragged lengths in [1024, 8192]) through the layer form"""
    _layer_case(qt, dev, 1004, 16, 4, 8192 + 8, 1024, 8192)
