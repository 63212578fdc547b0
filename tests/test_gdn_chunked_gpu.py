"""GPU parity of the chunked (C = 64) GatedDeltaNet prefill against the sequential CPU oracle.
Tolerance (the stated target): final state and outputs within 2e-3 relative of the sequential reference."""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from tests import chunk_pack as P
from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    q._lib.lib()
    return q


def gdn_inputs(seed, T, state_scale=0.02):
    """q, k (normalized), v, a, b as benchmark config 0 draws them, plus layer parameters and an initial state"""
    gen = torch.Generator().manual_seed(seed)
    cw, A_log, dtb, gw = layer_params(seed)
    q, k = O.normalize_qk(rand_bf(gen, (T, 16, 128)), rand_bf(gen, (T, 16, 128)))
    v, a, b = rand_bf(gen, (T, 16, 128)), rand_bf(gen, (T, 16)), rand_bf(gen, (T, 16))
    S0 = (torch.randn((16, 128, 128), generator=gen) * state_scale).numpy()
    return q, k, v, a, b, A_log, dtb, S0


@pytest.mark.parametrize("T", [64, 5, 100, 256])
def test_phase_b_on_reference_records(qt, dev, T):
    """phase B alone, fed with records packed on the CPU from the float64 chunk matrices"""
    q, k, v, a, b, A_log, dtb, S0 = gdn_inputs(40 + T, T)
    lg = O.log_decay(a, A_log, dtb)
    _, beta = O.gates(a, b, A_log, dtb)
    raw, ops, U, gC = P.chunk_records(q, k, v, lg, beta)
    y, s1 = qt.gdn_nax.phase_b(to_dev(q, dev, BF16), None, None, to_dev(ops.reshape(-1), dev), to_dev(U.reshape(-1), dev),
                               to_dev(gC.reshape(-1), dev), to_dev(S0[None], dev))
    oy, os_ = O.gated_delta_update(q[None], k[None], v[None], a[None], b[None], A_log, dtb, S0[None])
    check_rel("final state rel-L2", to_np(s1), os_, 2e-3, rel_l2)
    check_rel("final state max", to_np(s1), os_, 2e-3, rel_max)
    check_rel("y rel-L2", to_np(y), oy[0], 2e-3, rel_l2)


def proj_inputs(seed, T, scale=1.0, state_scale=0.02):
    gen = torch.Generator().manual_seed(seed)
    cw, A_log, dtb, gw = layer_params(seed)
    proj = rand_bf(gen, (T, PW), scale)
    cs = rand_bf(gen, (3, CD))
    S0 = (torch.randn((16, 128, 128), generator=gen) * state_scale).numpy()
    return proj, cs, cw, A_log, dtb, gw, S0


@pytest.mark.parametrize("T", [5, 64, 100])
def test_phase_a_records_vs_float64(qt, dev, T):
    """phase A's packed operands against the float64 chunk matrices (the fp16 operands carry 11 significant bits)"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(60 + T, T)
    q, k, v, ops, U, gC = qt.gdn_nax.prep_a(to_dev(proj, dev, BF16), to_dev(cs, dev, BF16), to_dev(cw, dev, BF16), to_dev(A_log, dev),
                                             to_dev(dtb, dev))
    oq, ok, ov = O.conv_prep(proj, cs, cw)
    check_equal("q", to_np(q), oq)                                            # bit-identical to conv_prep (tests/gdn_fuse.py:29-45)
    check_equal("k", to_np(k), ok)
    check_equal("v", to_np(v), ov)
    lg = O.log_decay(proj[:, 8208:8224], A_log, dtb)
    _, beta = O.gates(proj[:, 8208:8224], proj[:, 8192:8208], A_log, dtb)
    raw, rops, rU, rgC = P.chunk_records(oq, ok, ov, lg, beta)
    NC = (T + 63) // 64
    gops = to_np(ops).reshape(NC, 16, 28672).astype(np.float64)
    rops = rops.astype(np.float64)
    names = (("Wn", 0, 8192), ("Qg", 8192, 16384), ("Kd", 16384, 24576), ("Am", 24576, 28672))
    for name, lo, hi in names:
        for c in range(NC):
            for h in range(16):
                ref = rops[c, h, lo:hi]
                tol = 3e-3 * np.abs(ref).max() + 1.2e-7                    # + two fp16 subnormal steps (fast-decaying heads)
                d = np.abs(gops[c, h, lo:hi] - ref).max()
                if d > tol:
                    raise AssertionError(f"{name} chunk {c} head {h}: max abs diff {d:.3e} (scale {np.abs(ref).max():.3e})")
    check_rel("U", to_np(U).reshape(rU.shape), rU, 3e-3, rel_max)
    check_rel("gamma_C", to_np(gC).reshape(rgC.shape), rgC, 1e-5, rel_max)


@pytest.mark.parametrize("T", [5, 16, 37, 64, 65, 300])
def test_chunked_prefill_vs_sequential_oracle(qt, dev, T):
    """prep_a + phase_b + gated norm against the sequential restatement of the layer core (partial chunks as tests/gdn_fuse.py:29)"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(80 + T, T)
    dproj = to_dev(proj, dev, BF16)
    q, k, v, ops, U, gC = qt.gdn_nax.prep_a(dproj, to_dev(cs, dev, BF16), to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev))
    y, s1 = qt.gdn_nax.phase_b(q, k, v, ops, U, gC, to_dev(S0[None], dev))
    out = qt.prefill.gated_norm(y, dproj, to_dev(gw, dev))
    oo, oy, otail, os_ = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    check_rel("final state rel-L2", to_np(s1)[0], os_, 2e-3, rel_l2)
    check_rel("final state max", to_np(s1)[0], os_, 2e-3, rel_max)
    check_rel("y rel-L2", to_np(y).reshape(T, 2048), oy, 2e-3, rel_l2)
    check_rel("gated output rel-L2", to_np(out), oo, 2e-3, rel_l2)
    # gdn_chunked (q, k, v given) is the same computation
    y2, s2 = qt.gdn_nax.gdn_chunked(q, k, v, dproj, to_dev(A_log, dev), to_dev(dtb, dev), to_dev(S0[None], dev))
    check_tensors_equal("gdn_chunked y", y2, y)
    check_tensors_equal("gdn_chunked state", s2, s1)
    # the output kernel with the gated norm fused in gives the bits of the two separate kernels
    out3, s3 = qt.gdn_nax.phase_b_norm(dproj, ops, U, gC, to_dev(S0[None], dev), to_dev(gw, dev))
    check_tensors_equal("fused gated norm", out3, out)
    check_tensors_equal("fused gated norm state", s3, s1)


@pytest.mark.parametrize("T", [512, 2048])
def test_config2_chunked_prefill(qt, dev, T):
    """benchmark config 2: B=1, chunk 64, nonzero initial state ~N(0,0.02) (prefix-cache resume), conv first, gated norm last"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(1002, T)
    dproj = to_dev(proj, dev, BF16)
    q, k, v, ops, U, gC = qt.gdn_nax.prep_a(dproj, to_dev(cs, dev, BF16), to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev))
    y, s1 = qt.gdn_nax.phase_b(q, k, v, ops, U, gC, to_dev(S0[None], dev))
    out = qt.prefill.gated_norm(y, dproj, to_dev(gw, dev))
    oo, oy, otail, os_ = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    e1 = check_rel("final state rel-L2", to_np(s1)[0], os_, 2e-3, rel_l2)
    e2 = check_rel("y rel-L2", to_np(y).reshape(T, 2048), oy, 2e-3, rel_l2)
    e3 = check_rel("gated output rel-L2", to_np(out), oo, 2e-3, rel_l2)
    print(f"T={T}: state {e1:.2e}, y {e2:.2e}, out {e3:.2e}")
    # the layer core (fused output + norm kernel) returns the same bits, and the conv tail of prefill.py:262-263
    o4, conv4, s4 = qt.prefill.gdn_core(dproj, to_dev(cs[None], dev, BF16), to_dev(S0[None], dev), to_dev(cw, dev, BF16),
                                        to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev))
    check_tensors_equal("gdn_core output", o4, out)
    check_tensors_equal("gdn_core state", s4, s1)
    check_equal("gdn_core conv tail", to_np(conv4)[0], otail)


@pytest.mark.parametrize("T", [8192, 8131, 4100, 4033, 4032])
def test_config2_long_prefill(qt, dev, T):
    """config 2's longest sweep point (T = 8192: a chain of 128 chunks, each step rounding its operands to half precision), the
    same with a partial last chunk, 65 chunks (the output units of the one-launch form of phase B, which these lengths
    take, then run different numbers of rounds), and the two lengths either side of the switch between the forms (64 chunks,
    the last one of a single token: one launch; 63 chunks: two), from a nonzero state, through the layer core (reference entry
    qwen35/gdn_nax.py:413-426).  Run twice on the same buffers: the second launch finds the progress words the first one left.
    The per-head errors are checked too: a head whose state decays fast must not hide behind the slow ones."""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(2002 + T, T)
    o4, conv4, s4 = qt.prefill.gdn_core(to_dev(proj, dev, BF16), to_dev(cs[None], dev, BF16), to_dev(S0[None], dev), to_dev(cw, dev, BF16),
                                        to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev))
    o5, conv5, s5 = qt.prefill.gdn_core(to_dev(proj, dev, BF16), to_dev(cs[None], dev, BF16), to_dev(S0[None], dev), to_dev(cw, dev, BF16),
                                        to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev))
    check_tensors_equal("second launch, outputs", o5, o4)
    check_tensors_equal("second launch, state", s5, s4)
    oo, oy, otail, os_ = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    e1 = check_rel("final state rel-L2", to_np(s4)[0], os_, 2e-3, rel_l2)
    e2 = check_rel("final state max", to_np(s4)[0], os_, 2e-3, rel_max)
    e3 = check_rel("gated output rel-L2", to_np(o4), oo, 2e-3, rel_l2)
    got, ref = to_np(o4).reshape(T, 16, 128), oo.reshape(T, 16, 128)
    for h in range(16):
        check_rel(f"head {h} state rel-L2", to_np(s4)[0, h], os_[h], 2e-3, rel_l2)
        check_rel(f"head {h} output rel-L2", got[:, h], ref[:, h], 2e-3, rel_l2)
    for lo in range(0, T, 1024):                                              # no stretch of the sequence is worse than the bound
        check_rel(f"tokens {lo}.. output rel-L2", got[lo:lo + 1024], ref[lo:lo + 1024], 2e-3, rel_l2)
    check_equal("conv tail", to_np(conv4)[0], otail)
    # the launches left their progress words, queue head and done count zero, and no output workgroup gave up its wait
    flag_halves = qt._lib.lib().qt_gdn_chunk_snap_bytes(0) // 2
    for snap in qt.gdn_nax._SNAP.values():
        assert int(snap[:flag_halves].view(torch.int32).ne(0).sum().item()) == 0
    print(f"T={T}: state L2 {e1:.2e} max {e2:.2e}, out {e3:.2e}")


@pytest.mark.parametrize("T,state_scale", [(300, 0.3), (300, 1.0), (2048, 0.3), (2048, 1.0)])
def test_chunked_prefill_large_initial_state(qt, dev, T, state_scale):
    """initial states at the scales the reference's own tests draw (N(0,1) * 0.1 and * 0.3 in tests/gdn_fuse.py, bench/gdn_nax.py:25-30)
    and a unit-variance one: the half-precision operands of the chain must carry them"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(500 + T, T, state_scale=state_scale)
    o4, conv4, s4 = qt.prefill.gdn_core(to_dev(proj, dev, BF16), to_dev(cs[None], dev, BF16), to_dev(S0[None], dev), to_dev(cw, dev, BF16),
                                        to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev))
    oo, oy, otail, os_ = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    check_rel("final state rel-L2", to_np(s4)[0], os_, 2e-3, rel_l2)
    check_rel("final state max", to_np(s4)[0], os_, 2e-3, rel_max)
    check_rel("gated output rel-L2", to_np(o4), oo, 2e-3, rel_l2)
    check_rel("first chunk's gated output rel-L2", to_np(o4)[:64], oo[:64], 2e-3, rel_l2)


@pytest.mark.parametrize("T", [1, 2, 3, 5, 64, 65, 200])
def test_fused_conv_phase_a_equals_separate_kernels(qt, dev, T):
    """phase A fed by conv_prep's q, k, v and phase A convolving the projection rows itself give the same records, bit for bit;
    the conv window it leaves is the last three input rows (qwen35/prefill.py:262-263), also when S < 3"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(300 + T, T)
    dproj, dcs, dcw, dA, ddt = to_dev(proj, dev, BF16), to_dev(cs, dev, BF16), to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev)
    q, k, v = qt.prefill.conv_prep(dproj, dcs, dcw)
    _, _, _, ops0, U0, gC0 = qt.gdn_nax._phase_a(dproj, None, None, dA, ddt, qkv=(q, k, v))
    tail = torch.zeros((3, CD), dtype=BF16, device=dev)
    q1, k1, v1, ops1, U1, gC1 = qt.gdn_nax._phase_a(dproj, dcs, dcw, dA, ddt, conv_out=tail)
    _, _, _, ops2, U2, gC2 = qt.gdn_nax._phase_a(dproj, dcs, dcw, dA, ddt, want_qkv=False)
    for name, a, b in (("q", q1, q), ("k", k1, k), ("v", v1, v), ("ops", ops1, ops0), ("U", U1, U0), ("gC", gC1, gC0),
                       ("ops (no q, k, v stored)", ops2, ops0), ("U (no q, k, v stored)", U2, U0), ("gC (no q, k, v stored)", gC2, gC0)):
        check_tensors_equal(name, a, b)
    check_equal("conv tail", to_np(tail), np.concatenate([cs, proj[:, :CD]], axis=0)[-3:])


def test_fused_conv_silu_exhaustive(qt, dev):
    """every finite bf16 value as a conv sum (taps 0, 0, 0, 1) through the fused conv of phase A: the SiLU table and what
    lies outside it, against the restatement of silu_bf16 (mslib.py:21-22)"""
    f = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    x = f[np.isfinite(f)]
    S = 32
    gen = torch.Generator().manual_seed(7)
    proj = rand_bf(gen, (S, PW))
    vals = np.resize(x, S * 2048).reshape(S, 2048)
    proj[:, 4096:6144] = vals
    cw, A_log, dtb, gw = layer_params(3)
    cw[4096:6144] = (0.0, 0.0, 0.0, 1.0)
    q, k, v, ops, U, gC = qt.gdn_nax.prep_a(to_dev(proj, dev, BF16), torch.zeros((3, CD), dtype=BF16, device=dev), to_dev(cw, dev, BF16),
                                             to_dev(A_log, dev), to_dev(dtb, dev))
    got, ref = to_np(v).reshape(S, 2048), O.silu_bf16(vals)
    check_equal("silu of every finite bf16 value", got, ref)
    nz = vals != 0                                                            # (a conv sum of zeros is +0 whatever the sign of x)
    assert np.array_equal(np.signbit(got[nz]), np.signbit(ref[nz])), "sign of a zero result"
    q2, k2, v2 = qt.prefill.conv_prep(to_dev(proj, dev, BF16), torch.zeros((3, CD), dtype=BF16, device=dev), to_dev(cw, dev, BF16))
    check_tensors_equal("conv_prep v", v2, v)
    check_tensors_equal("conv_prep q", q2, q)
    check_tensors_equal("conv_prep k", k2, k)


def _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0):
    return qt.prefill.gdn_core(to_dev(proj, dev, BF16), to_dev(cs[None], dev, BF16), to_dev(S0[None], dev), to_dev(cw, dev, BF16),
                               to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev))


@pytest.mark.parametrize("T", [300, 4100])
def test_chunked_prefill_at_the_edge_of_the_half_precision_range(qt, dev, T):
    """the documented operand range (|v|, |S| up to 65504): a state of N(0, 1e4) (largest element ~4.8e4) and conv outputs of a few
    thousand keep the 2e-3 tolerance, in both launch forms of phase B, and leave the status word clear"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(900 + T, T, state_scale=1.0e4)
    proj[:, 4096:6144] = bf(proj[:, 4096:6144] * 2000.0)
    assert np.abs(S0).max() < 6.0e4
    o4, conv4, s4 = _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0)
    qt.gdn_nax.check_status(dev, sync=True)
    oo, oy, otail, os_ = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    assert 1.0e3 < np.abs(oy).max() < 6.0e4
    check_rel("final state rel-L2", to_np(s4)[0], os_, 2e-3, rel_l2)
    check_rel("final state max", to_np(s4)[0], os_, 2e-3, rel_max)
    check_rel("gated output rel-L2", to_np(o4), oo, 2e-3, rel_l2)


@pytest.mark.parametrize("T", [300, 4100])
def test_status_word_reports_operands_beyond_half_precision(qt, dev, T):
    """a state beyond 65504 cannot be carried by the half-precision operands: the launch ends normally, bit 1 of the status
    word is set, and the wrapper raises at the next call (or at check_status) instead of handing out the rows; the word is
    reset by the raise, so the launch after it runs clean"""
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(950 + T, T, state_scale=1.0e6)
    _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0)
    with pytest.raises(qt.gdn_nax.ChunkedPrefillError, match="not finite"):
        qt.gdn_nax.check_status(dev, sync=True)
    qt.gdn_nax.check_status(dev, sync=True)                                   # reset
    _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0)
    torch.cuda.synchronize()                                                  # the read-back behind the launch has landed:
    with pytest.raises(qt.gdn_nax.ChunkedPrefillError):                       # the next call sees it without waiting
        _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0 * 1e-8)
    o4, conv4, s4 = _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0 * 1e-8)
    qt.gdn_nax.check_status(dev, sync=True)
    oo, oy, otail, os_ = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0 * 1e-8, gw)
    check_rel("gated output after the reset", to_np(o4), oo, 2e-3, rel_l2)


def test_give_up_path_ends_the_launch_and_leaves_the_flags_clean(qt, dev):
    """the bounded wait of the one-launch form, forced from the host with a poll limit of one: output workgroups give up on chunks
    the chain has not published yet, leave those rows unwritten and set bit 0 of the status word; every workgroup ends, the
    last one to finish (a chain workgroup here: the output workgroups are done long before it) clears the progress words, and
    the next launch on the same buffer, with the default limit, gives the bits of an undisturbed one"""
    T = 8192
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(2002 + T, T)
    want, _, s_want = _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0)
    qt.gdn_nax.check_status(dev, sync=True)
    lib = qt._lib.lib()
    assert lib.qt_gdn_phase_b_poll_limit(1) == 0
    try:
        _, _, s_gave_up = _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0)
        torch.cuda.synchronize()
    finally:
        assert lib.qt_gdn_phase_b_poll_limit(0) == 0
    check_tensors_equal("the chain is not affected by output workgroups that gave up", s_gave_up, s_want)
    flag_halves = lib.qt_gdn_chunk_snap_bytes(0) // 2
    off = lib.qt_gdn_chunk_status_offset() // 4
    for snap in qt.gdn_nax._SNAP.values():
        words = snap[:flag_halves].view(torch.int32).clone()
        assert int(words[off].item()) & qt.gdn_nax.GAVE_UP
        words[off] = 0
        assert int(words.ne(0).sum().item()) == 0, "progress words, done count or queue head left set"
    with pytest.raises(qt.gdn_nax.ChunkedPrefillError, match="gave up"):
        qt.gdn_nax.check_status(dev, sync=True)
    got, _, s_got = _core(qt, dev, proj, cs, cw, A_log, dtb, gw, S0)
    qt.gdn_nax.check_status(dev, sync=True)
    check_tensors_equal("outputs of the launch after a give-up", got, want)
    check_tensors_equal("state of the launch after a give-up", s_got, s_want)


@pytest.mark.parametrize("T", [4096, 4100])
def test_phase_b_through_the_c_abi_with_a_caller_owned_snap(qt, dev, T):
    """qt_gdn_phase_b_norm called directly (ctypes) with a snap buffer the caller allocated and zeroed once: two launches in a row
    give the bits of the wrapper path, and the flag area is zero after each"""
    import ctypes
    proj, cs, cw, A_log, dtb, gw, S0 = proj_inputs(3000 + T, T)
    dproj, dgw, dS0 = to_dev(proj, dev, BF16), to_dev(gw, dev), to_dev(S0[None], dev)
    _, _, _, ops, U, gC = qt.gdn_nax._phase_a(dproj, to_dev(cs, dev, BF16), to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev),
                                              want_qkv=False)
    want, s_want = qt.gdn_nax.phase_b_norm(dproj, ops, U, gC, dS0, dgw)
    lib = qt._lib.lib()
    nbytes = lib.qt_gdn_chunk_snap_bytes(T)
    flag_bytes = lib.qt_gdn_chunk_snap_bytes(0)
    snap = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    snap.fill_(0xAB)                                                          # snapshots may hold anything ...
    snap[:flag_bytes].zero_()                                                 # ... the flag area must be zero
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for launch in range(2):
        out = torch.empty((T, 2048), dtype=BF16, device=dev)
        s1 = torch.empty_like(dS0)
        rc = lib.qt_gdn_phase_b_norm(p(ops), p(U), p(gC), p(snap), p(dS0), p(s1), p(dproj), p(dgw), 1e-6, p(out), T, stream)
        assert rc == 0
        torch.cuda.synchronize()
        check_tensors_equal(f"launch {launch}: outputs", out, want)
        check_tensors_equal(f"launch {launch}: state", s1, s_want)
        assert int(snap[:flag_bytes].ne(0).sum().item()) == 0, "flag area (status word included) not zero after the launch"
