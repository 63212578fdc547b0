"""GPU parity of the fused GatedDeltaNet decode / verify step and its stand-alone pieces against the CPU oracle.

Tolerances (the stated target): fp32 state within 1e-4 relative per decode step; everything the elementwise prologue
produces (conv windows, q, k, v, gates, gated norm) is bit-exact by construction of the arithmetic contract; bf16 outputs
of float32 dot products within 1 bf16 ulp."""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from oracle import c_oracle as C
from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    q._lib.lib()
    return q


def all_bf16():
    f = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    return f[np.isfinite(f)]


# ------------------------------------------------------------------------------------- scalar helpers, exhaustively
def test_sigmoid_softplus_exhaustive(qt, dev):
    x = all_bf16()
    x = x[np.abs(x) < 1e30]
    n = (len(x) // 16) * 16
    x = x[:n].reshape(-1, 16)
    a = to_dev(x, dev, BF16)
    A0 = torch.zeros(16, device=dev)
    g, lg, beta = qt.gated_delta._gates(A0, a, a, A0, want_lg=True)
    check_equal('np.array_equal(to_np(beta), O.sigmoid_bf16(x))', to_np(beta), O.sigmoid_bf16(x))
    check_equal('np.array_equal(-to_np(lg), O.softplus_bf16(x))', -to_np(lg), O.softplus_bf16(x))
    og, _ = O.gates(x, x, np.zeros(16, np.float32), np.zeros(16, np.float32))
    check_rel('g (float exp, not rounded to bf16)', to_np(g), og, 4e-7, lambda a, b: float(np.max(np.abs(a - b) / np.maximum(b, 1e-30))))


def test_silu_exhaustive_through_conv(qt, dev):
    x = all_bf16()
    x = x[np.abs(x) < 1e30]
    S = 32
    proj = np.zeros((S, PW), np.float32)
    vals = np.resize(x, S * 2048).reshape(S, 2048)
    proj[:, 4096:6144] = vals
    cw = np.zeros((CD, 4), np.float32)
    cw[:, 3] = 1.0
    q, k, v = qt.prefill.conv_prep(to_dev(proj, dev, BF16), torch.zeros((3, CD), dtype=BF16, device=dev), to_dev(cw, dev, BF16))
    check_equal('np.array_equal(to_np(v).reshape(S, 2048), O.silu_b', to_np(v).reshape(S, 2048), O.silu_bf16(vals))


# ------------------------------------------------------------------------------------- stand-alone pieces
@pytest.mark.parametrize("S", [1, 2, 5, 37, 300, 2048])
def test_conv_prep_bit_exact(qt, dev, S):
    gen = torch.Generator().manual_seed(100 + S)
    cw, A_log, dtb, gw = layer_params(1)
    proj = rand_bf(gen, (S, PW), 1.5)
    cs = rand_bf(gen, (3, CD))
    q, k, v = qt.prefill.conv_prep(to_dev(proj, dev, BF16), to_dev(cs, dev, BF16), to_dev(cw, dev, BF16).reshape(CD, 4, 1))
    oq, ok, ov = O.conv_prep(proj, cs, cw)
    check_equal('np.array_equal(to_np(q), oq)', to_np(q), oq)
    check_equal('np.array_equal(to_np(k), ok)', to_np(k), ok)
    check_equal('np.array_equal(to_np(v), ov)', to_np(v), ov)


@pytest.mark.parametrize("B,T", [(2, 5), (4, 512)])               # the larger one: millions of values, for the one-in-10^5 cases
def test_normalize_qk_and_compute_g_bit_exact(qt, dev, B, T):
    gen = torch.Generator().manual_seed(7 + T)
    cw, A_log, dtb, gw = layer_params(2)
    q = rand_bf(gen, (B, T, 16, 128), 2)
    k = rand_bf(gen, (B, T, 16, 128), 2)
    qn, kn = qt.gated_delta.normalize_qk(to_dev(q, dev, BF16), to_dev(k, dev, BF16), inv_scale=128 ** -0.5, eps=1e-6)
    oq, ok = O.normalize_qk(q, k)
    check_equal('np.array_equal(to_np(qn), oq)', to_np(qn), oq)
    check_equal('np.array_equal(to_np(kn), ok)', to_np(kn), ok)
    a = rand_bf(gen, (B, T, 16), 2)
    g = qt.gated_delta.compute_g(to_dev(A_log, dev), to_dev(a, dev, BF16), to_dev(dtb, dev, BF16))
    og, _ = O.gates(a, a, A_log, dtb)
    assert g.dtype == torch.float32
    check_rel('g', to_np(g), og, 1e-6, lambda a, b: float(np.max(np.abs(a - b) / np.maximum(b, 1e-30))))
    with pytest.raises(ValueError):
        qt.gated_delta.normalize_qk(to_dev(q[..., :64], dev, BF16), to_dev(k[..., :64], dev, BF16), inv_scale=64 ** -0.5, eps=1e-6)


@pytest.mark.parametrize("R", [1, 7, 64, 2048, 4099])
def test_gated_norm_bit_exact(qt, dev, R):
    gen = torch.Generator().manual_seed(200 + R)
    cw, A_log, dtb, gw = layer_params(3)
    y = rand_bf(gen, (R, 2048), 3)
    proj = rand_bf(gen, (R, PW), 2)
    o1 = qt.batch.gnorm_rows(to_dev(y, dev, BF16), to_dev(proj, dev, BF16), to_dev(gw, dev))
    o2 = qt.prefill.gated_norm(to_dev(y, dev, BF16).reshape(R, 16, 128), to_dev(proj, dev, BF16), to_dev(gw, dev))
    ref = O.gated_norm(y, proj, gw)
    check_equal('np.array_equal(to_np(o1), ref)', to_np(o1), ref)
    check_equal('np.array_equal(to_np(o2), ref)', to_np(o2), ref)


# ------------------------------------------------------------------------------------- the sequential recurrence
@pytest.mark.parametrize("B,T", [(1, 1), (1, 3), (2, 5), (4, 1), (1, 257)])
def test_gated_delta_update_vs_oracle(qt, dev, B, T):
    """shapes of the reference's tests/gated_delta.py:44-58: inputs N(0,1)*2 bf16, state N(0,1)*0.1"""
    gen = torch.Generator().manual_seed(B * 1000 + T)
    cw, A_log, dtb, gw = layer_params(4)
    q, k = rand_bf(gen, (B, T, 16, 128), 2), rand_bf(gen, (B, T, 16, 128), 2)
    v, a, b = rand_bf(gen, (B, T, 16, 128)), rand_bf(gen, (B, T, 16)), rand_bf(gen, (B, T, 16))
    st = (torch.randn((B, 16, 128, 128), generator=gen) * 0.1).numpy()
    qn, kn = O.normalize_qk(q, k)
    d = lambda x: to_dev(x, dev, BF16)
    y, s = qt.gated_delta.gated_delta_update(d(qn), d(kn), d(v), d(a), d(b), to_dev(A_log, dev), d(dtb), to_dev(st, dev))
    oy, os_ = O.gated_delta_update(qn, kn, v, a, b, A_log, dtb, st)
    check_rel('to_np(s), os_', to_np(s), os_, 1e-4, rel_max)
    check_rel('to_np(s), os_', to_np(s), os_, 1e-5, rel_l2)
    check_ulp('to_np(y)', to_np(y), oy)
    assert (to_np(y) != oy).mean() < 0.02
    y0, s0 = qt.gated_delta.gated_delta_update(d(qn), d(kn), d(v), d(a), d(b), to_dev(A_log, dev), d(dtb))
    yz, sz = qt.gated_delta.gated_delta_update(d(qn), d(kn), d(v), d(a), d(b), to_dev(A_log, dev), d(dtb),
                                               torch.zeros((B, 16, 128, 128), device=dev))
    check_tensors_equal('torch.equal(y0, yz)', y0, yz)
    check_tensors_equal('torch.equal(s0, sz)', s0, sz)


def test_gated_delta_update_gqa_heads_and_errors(qt, dev):
    gen = torch.Generator().manual_seed(5)
    cw, A_log, dtb, gw = layer_params(5)
    B, T = 2, 4
    q, k = O.normalize_qk(rand_bf(gen, (B, T, 8, 128)), rand_bf(gen, (B, T, 8, 128)))
    v, a, b = rand_bf(gen, (B, T, 16, 64)), rand_bf(gen, (B, T, 16)), rand_bf(gen, (B, T, 16))
    d = lambda x: to_dev(x, dev, BF16)
    y, s = qt.gated_delta.gated_delta_update(d(q), d(k), d(v), d(a), d(b), to_dev(A_log, dev), d(dtb))
    oy, os_ = O.gated_delta_update(q, k, v, a, b, A_log, dtb)
    check_rel('to_np(s), os_', to_np(s), os_, 1e-4, rel_max)
    check_ulp('to_np(y)', to_np(y), oy)
    with pytest.raises(ValueError):                                            # gated_delta.py:164-166
        qt.gated_delta.gated_delta_update(d(q[..., :64]), d(k[..., :64]), d(v), d(a), d(b), to_dev(A_log, dev), d(dtb))


@pytest.mark.parametrize("Dv", [8, 24, 72])
def test_gated_delta_update_value_dim_multiple_of_8(qt, dev, Dv):
    """the reference takes every value dim that is a multiple of 8 (qwen35/gated_delta.py:164-166), not only multiples of 16"""
    gen = torch.Generator().manual_seed(300 + Dv)
    cw, A_log, dtb, gw = layer_params(13)
    B, T, H = 2, 7, 4
    q, k = O.normalize_qk(rand_bf(gen, (B, T, H, 128)), rand_bf(gen, (B, T, H, 128)))
    v, a, b = rand_bf(gen, (B, T, H, Dv)), rand_bf(gen, (B, T, H)), rand_bf(gen, (B, T, H))
    S0 = (torch.randn((B, H, Dv, 128), generator=gen) * 0.1).numpy()
    y, s1 = qt.gated_delta.gated_delta_update(to_dev(q, dev, BF16), to_dev(k, dev, BF16), to_dev(v, dev, BF16), to_dev(a, dev, BF16),
                                              to_dev(b, dev, BF16), to_dev(A_log[:H], dev), to_dev(dtb[:H], dev), to_dev(S0, dev))
    oy, os_ = O.gated_delta_update(q, k, v, a, b, A_log[:H], dtb[:H], S0)
    check_rel("state", to_np(s1), os_, 1e-4, rel_max)
    check_ulp("y", to_np(y), oy)
    with pytest.raises(ValueError):
        qt.gated_delta.gated_delta_update(to_dev(q, dev, BF16), to_dev(k, dev, BF16), to_dev(rand_bf(gen, (B, T, H, 12)), dev, BF16),
                                          to_dev(a, dev, BF16), to_dev(b, dev, BF16), to_dev(A_log[:H], dev), to_dev(dtb[:H], dev))


def test_config0_token_by_token(qt, dev):
    """benchmark config 0: one layer, B=1, T=256 run token by token from a zero state; per-step state error <= 1e-4."""
    gen = torch.Generator().manual_seed(1000)
    T = 256
    A_log = (torch.rand(16, generator=gen) * 2.7).numpy()
    dtb = (torch.randn(16, generator=gen) * 0.1).bfloat16().float().numpy()
    q, k = O.normalize_qk(rand_bf(gen, (1, T, 16, 128)), rand_bf(gen, (1, T, 16, 128)))
    v, a, b = rand_bf(gen, (1, T, 16, 128)), rand_bf(gen, (1, T, 16)), rand_bf(gen, (1, T, 16))
    d = lambda x: to_dev(x, dev, BF16)
    dq, dk, dv, da, db = d(q), d(k), d(v), d(a), d(b)
    dA, ddt = to_dev(A_log, dev), d(dtb)
    s = torch.zeros((1, 16, 128, 128), device=dev)
    so = np.zeros((1, 16, 128, 128), np.float32)
    worst = 0.0
    for t in range(T):
        y, s = qt.gated_delta.gated_delta_update(dq[:, t:t + 1].contiguous(), dk[:, t:t + 1].contiguous(), dv[:, t:t + 1].contiguous(),
                                                 da[:, t:t + 1].contiguous(), db[:, t:t + 1].contiguous(), dA, ddt, s)
        oy, so = O.gated_delta_update(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], a[:, t:t + 1], b[:, t:t + 1], A_log, dtb, so)
        worst = max(worst, rel_max(to_np(s), so))
        check_ulp('to_np(y)', to_np(y), oy)
    assert worst <= 1e-4, worst
    # the whole sequence in one call is bitwise the chained single-token calls
    y_all, s_all = qt.gated_delta.gated_delta_update(dq, dk, dv, da, db, dA, ddt)
    check_tensors_equal('torch.equal(s_all, s)', s_all, s)


# ------------------------------------------------------------------------------------- fused step
def _solo(qt, dev, proj, cs, cw, A_log, dtb, ss, sel, **kw):
    return qt.kernels.deltanet(to_dev(proj, dev, BF16), to_dev(cs, dev, BF16), to_dev(cw, dev, BF16), to_dev(A_log, dev),
                               to_dev(dtb, dev), to_dev(ss, dev), torch.tensor([sel], dtype=torch.int32, device=dev), **kw)


@pytest.mark.parametrize("M", [1, 3, 4, 8, 16])                             # (16: the most the entry point takes)
def test_deltanet_solo_vs_oracle_and_chaining(qt, dev, M):
    gen = torch.Generator().manual_seed(300 + M)
    cw, A_log, dtb, gw = layer_params(6)
    proj = rand_bf(gen, (M, PW), 1.5)
    cs = rand_bf(gen, (4, 3, CD))
    ss = (torch.randn((4, 16, 128, 128), generator=gen) * 0.1).numpy()
    y, c, s = _solo(qt, dev, proj, cs, cw, A_log, dtb, ss, 2)
    oy, oc, os_ = O.deltanet(proj, cs, cw, A_log, dtb, ss, np.array([2]))
    check_equal('conv snapshots', to_np(c), oc)                                # bit exact
    check_rel('to_np(s), os_', to_np(s), os_, 1e-4, rel_max)
    check_rel('to_np(s), os_', to_np(s), os_, 1e-5, rel_l2)
    check_ulp('to_np(y)', to_np(y), oy)
    # M tokens == M single-token calls, bitwise (reference tests/verify.py:28-33)
    c1, s1 = to_dev(cs[2:3], dev, BF16), to_dev(ss[2:3], dev)
    sel0 = torch.zeros(1, dtype=torch.int32, device=dev)
    for j in range(M):
        yj, c1, s1 = qt.kernels.deltanet(to_dev(proj[j:j + 1], dev, BF16), c1, to_dev(cw, dev, BF16), to_dev(A_log, dev),
                                         to_dev(dtb, dev), s1, sel0)
        check_tensors_equal('torch.equal(yj[0], y[j])', yj[0], y[j])
        check_tensors_equal('torch.equal(c1[0], c[j])', c1[0], c[j])
        check_tensors_equal('torch.equal(s1[0], s[j])', s1[0], s[j])
    # every workgroup split gives the same bits
    for rows in (16, 32, 64, 128):
        y2, c2, s2 = _solo(qt, dev, proj, cs, cw, A_log, dtb, ss, 2, rows_per_wg=rows)
        check_tensors_equal('torch.equal(y2, y)', y2, y)
        check_tensors_equal('torch.equal(c2, c)', c2, c)
        check_tensors_equal('torch.equal(s2, s)', s2, s)


def test_fused_step_equals_separate_pieces(qt, dev):
    """deltanet == conv_prep + gated_delta_update on the GPU, bitwise"""
    gen = torch.Generator().manual_seed(9)
    cw, A_log, dtb, gw = layer_params(7)
    M = 4
    proj = to_dev(rand_bf(gen, (M, PW), 1.5), dev, BF16)
    cs = to_dev(rand_bf(gen, (1, 3, CD)), dev, BF16)
    ss = to_dev((torch.randn((1, 16, 128, 128), generator=gen) * 0.1).numpy(), dev)
    dcw, dA, ddt = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev)
    y, c, s = qt.kernels.deltanet(proj, cs, dcw, dA, ddt, ss, torch.zeros(1, dtype=torch.int32, device=dev))
    q, k, v = qt.prefill.conv_prep(proj, cs[0], dcw)
    y2, s2 = qt.gated_delta.gated_delta_update(q[None], k[None], v[None], proj[None, :, 8208:8224], proj[None, :, 8192:8208],
                                               dA, ddt, ss)
    check_tensors_equal('torch.equal(y2[0].reshape(M, 2048), y)', y2[0].reshape(M, 2048), y)
    check_tensors_equal('torch.equal(s2[0], s[-1])', s2[0], s[-1])


def test_deltanet_b_layout_of_reference_test(qt, dev):
    """reference tests/batch.py:42-71: 5 rows on slots scattered in a 7-slot pool, ragged positions"""
    rng = np.random.default_rng(11)
    cw, A_log, dtb, gw = layer_params(8)
    S, B = 6, 5
    slots = np.array([3, 0, 5, 1, 2], np.int32)
    pos = np.array([0, 1, 7, 100, 2047], np.int32)
    proj = bf(rng.standard_normal((B, PW)) * 2)
    cv = bf(rng.standard_normal((S + 1, 3, CD)))
    ssm0 = (rng.standard_normal((S + 1, 16, 128, 128)) * 0.3).astype(np.float32)
    cp = np.zeros(((S + 1) * 2, 3, CD), np.float32)
    for b in range(B):
        cp[slots[b] * 2 + (pos[b] & 1)] = cv[slots[b]]
    conv_pool, ssm_pool = to_dev(cp, dev, BF16), to_dev(ssm0, dev)
    dcw, dA, ddt = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev)
    y = qt.batch.deltanet_b(to_dev(proj, dev, BF16), conv_pool, dcw, dA, ddt, ssm_pool, to_dev(slots, dev), to_dev(pos, dev))
    ocp, ossm = cp.copy(), ssm0.copy()
    oy = O.deltanet_b(proj, ocp, cw, A_log, dtb, ossm, slots, pos)
    check_equal('conv pool', to_np(conv_pool), ocp)                            # windows, parity buffers, untouched buffers
    check_rel('to_np(ssm_pool), ossm', to_np(ssm_pool), ossm, 1e-4, rel_max)
    check_ulp('to_np(y)', to_np(y), oy)
    sel0 = torch.zeros(1, dtype=torch.int32, device=dev)
    for b in range(B):                                                         # batched == solo, bitwise
        s_ = int(slots[b])
        ry, rc, rs = qt.kernels.deltanet(to_dev(proj[b:b + 1], dev, BF16), to_dev(cv[s_:s_ + 1], dev, BF16), dcw, dA, ddt,
                                         to_dev(ssm0[s_:s_ + 1], dev), sel0)
        check_tensors_equal('torch.equal(y[b:b + 1], ry)', y[b:b + 1], ry)
        check_tensors_equal('torch.equal(ssm_pool[s_:s_ + 1], rs)', ssm_pool[s_:s_ + 1], rs)
        check_tensors_equal('torch.equal(conv_pool[s_ * 2 + ((int(pos[b]) & 1) ', conv_pool[s_ * 2 + ((int(pos[b]) & 1) ^ 1)][None], rc)
    check_equal('np.array_equal(to_np(ssm_pool[4]), ssm0[4])', to_np(ssm_pool[4]), ssm0[4])
    check_equal('np.array_equal(to_np(ssm_pool[6]), ssm0[6])', to_np(ssm_pool[6]), ssm0[6])
    # every workgroup shape (a head split over 8..1 workgroups, 2 or 4 whole heads per workgroup) gives the same bits
    for rows in (16, 32, 64, 128, 256, 512):
        cp2, ssm2 = to_dev(cp, dev, BF16), to_dev(ssm0, dev)
        y2 = qt.batch.deltanet_b(to_dev(proj, dev, BF16), cp2, dcw, dA, ddt, ssm2, to_dev(slots, dev), to_dev(pos, dev), rows_per_wg=rows)
        check_tensors_equal(f'y rows_per_wg={rows}', y2, y)
        check_tensors_equal(f'conv pool rows_per_wg={rows}', cp2, conv_pool)
        check_tensors_equal(f'ssm pool rows_per_wg={rows}', ssm2, ssm_pool)


@pytest.mark.parametrize("B", [1, 16, 24, 48, 64, 96])              # (every default workgroup shape: split head, 1, 2, 4 heads, half heads)
def test_deltanet_b_config1_steps(qt, dev, B):
    """benchmark config 1 (B = 1, 16, 64, and sizes between and beyond that take the other default shapes): consecutive steps with advancing positions; state ~ N(0,0.02).  The C oracle steps
    alongside from its own state (free running) and must stay within 1e-4 relative at every step."""
    gen = torch.Generator().manual_seed(1001)
    cw, A_log, dtb, gw = layer_params(9)
    steps = 12
    ssm = (torch.randn((B + 1, 16, 128, 128), generator=gen) * 0.02).numpy()
    cp = rand_bf(gen, ((B + 1) * 2, 3, CD))
    slots = torch.randperm(B, generator=gen).numpy().astype(np.int32)
    pos = torch.randint(0, 1000, (B,), generator=gen).numpy().astype(np.int32)
    conv_pool, ssm_pool = to_dev(cp, dev, BF16), to_dev(ssm, dev)
    dcw, dA, ddt = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev)
    ocp, ossm = C.to_bf16_bits(cp), ssm.copy()
    cwb = C.to_bf16_bits(cw).reshape(-1)
    for step in range(steps):
        proj = rand_bf(gen, (B, PW))
        y = qt.batch.deltanet_b(to_dev(proj, dev, BF16), conv_pool, dcw, dA, ddt, ssm_pool, to_dev(slots, dev), to_dev(pos, dev))
        oy = C.from_bf16_bits(C.decode_step(C.to_bf16_bits(proj), ocp, cwb, A_log, dtb, ossm, slots, pos, acc64=True, nthreads=8))
        got = to_np(ssm_pool)
        for b in range(B):
            check_rel('got[slots[b]], ossm[slots[b]]', got[slots[b]], ossm[slots[b]], 1e-4, rel_max)
        check_equal('np.array_equal(to_np(conv_pool), C.from_bf16_bits(', to_np(conv_pool), C.from_bf16_bits(ocp))
        check_ulp('to_np(y)', to_np(y), oy)
        check_equal('trash slot', got[B], ssm[B])                              # no row points at it here: untouched
        pos = pos + 1


def test_deltanet_b_out_of_range_slot_is_skipped(qt, dev):
    gen = torch.Generator().manual_seed(3)
    cw, A_log, dtb, gw = layer_params(10)
    ssm = to_dev((torch.randn((3, 16, 128, 128), generator=gen) * 0.02).numpy(), dev)
    conv = to_dev(rand_bf(gen, (6, 3, CD)), dev, BF16)
    s0, c0 = ssm.clone(), conv.clone()
    proj = to_dev(rand_bf(gen, (2, PW)), dev, BF16)
    qt.batch.deltanet_b(proj, conv, to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), ssm,
                        torch.tensor([7, -1], dtype=torch.int32, device=dev), torch.tensor([0, 0], dtype=torch.int32, device=dev))
    for rows in (256, 512):
        qt.batch.deltanet_b(proj, conv, to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), ssm,
                            torch.tensor([7, -1], dtype=torch.int32, device=dev), torch.tensor([0, 0], dtype=torch.int32, device=dev),
                            rows_per_wg=rows)
    torch.cuda.synchronize()
    check_tensors_equal('torch.equal(ssm, s0)', ssm, s0)
    check_tensors_equal('torch.equal(conv, c0)', conv, c0)


def test_deltanet_bm_layout_of_reference_test(qt, dev):
    """reference tests/batch_spec.py:40-67: 4 sequences, ragged entries / start snapshots / conv buffers, M = 3; config 4's M = 4;
    and M = 8, beyond what the reference's scheduler drafts"""
    for M, seed in ((3, 0), (4, 1004), (8, 1008)):
        rng = np.random.default_rng(seed)
        cw, A_log, dtb, gw = layer_params(11)
        NS, B = 6, 4
        sslots = np.array([4, 1, 5, 0], np.int32)
        sels = np.array([2, 0, 1, 2], np.int32)
        pars = np.array([1, 0, 0, 1], np.int32)
        cp = bf(rng.standard_normal(((NS + 1) * 2, M, 3, CD)))
        sp = (rng.standard_normal((NS + 1, M, 16, 128, 128)) * 0.1).astype(np.float32)
        proj = bf(rng.standard_normal((B * M, PW)) * 1.5)
        conv_pool, ssm_pool = to_dev(cp, dev, BF16), to_dev(sp, dev)
        dcw, dA, ddt = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev)
        y = qt.batch_spec.deltanet_bm(to_dev(proj, dev, BF16), conv_pool, dcw, dA, ddt, ssm_pool, to_dev(sslots, dev),
                                      to_dev(sels, dev), to_dev(pars, dev), M)
        ocp, osp = cp.copy(), sp.copy()
        oy = O.deltanet_bm(proj, ocp, cw, A_log, dtb, osp, sslots, sels, pars, M)
        check_equal('np.array_equal(to_np(conv_pool), ocp)', to_np(conv_pool), ocp)
        check_rel('to_np(ssm_pool), osp', to_np(ssm_pool), osp, 1e-4, rel_max)
        check_ulp('to_np(y)', to_np(y), oy)
        for b in range(B):                                                     # == solo deltanet(M) per sequence, bitwise
            s_, sl, pr = int(sslots[b]), int(sels[b]), int(pars[b])
            yr, cr, sr = qt.kernels.deltanet(to_dev(proj[b * M:(b + 1) * M], dev, BF16), to_dev(cp[s_ * 2 + pr], dev, BF16), dcw,
                                             dA, ddt, to_dev(sp[s_], dev), torch.tensor([sl], dtype=torch.int32, device=dev))
            check_tensors_equal('torch.equal(y[b * M:(b + 1) * M], yr)', y[b * M:(b + 1) * M], yr)
            check_tensors_equal('torch.equal(conv_pool[s_ * 2 + (pr ^ 1)], cr)', conv_pool[s_ * 2 + (pr ^ 1)], cr)
            check_tensors_equal('torch.equal(ssm_pool[s_], sr)', ssm_pool[s_], sr)
        for e in (2, 3, 6):
            check_equal('np.array_equal(to_np(ssm_pool[e]), sp[e])', to_np(ssm_pool[e]), sp[e])


@pytest.mark.parametrize("B", [16, 64])
def test_deltanet_b_config1_thousand_steps(qt, dev, B):
    """benchmark config 1 at its stated length: B slots, 1000 consecutive steps.  The C oracle (float64 dot products) runs
    free from its own state; y within one bf16 ulp at EVERY step, conv windows bit-exact, state within 1e-4 relative (so the
    kernel's float32 re-association y = g (S.q) + delta (k.q) is observed over the whole run, not over a dozen steps).  The
    state is compared at every step for B = 16 and at steps 1, 2, 5, 10, 50, 100, 500, 1000 for B = 64 (the headline's batch:
    65 MiB of state per comparison)."""
    steps = 1000
    state_at = set(range(steps)) if B == 16 else {0, 1, 4, 9, 49, 99, 499, 999}
    gen = torch.Generator().manual_seed(1001)
    cw, A_log, dtb, gw = layer_params(9)
    ssm = (torch.randn((B + 1, 16, 128, 128), generator=gen) * 0.02).numpy()
    cp = rand_bf(gen, ((B + 1) * 2, 3, CD))
    slots = torch.randperm(B, generator=gen).numpy().astype(np.int32)
    pos = torch.randint(0, 1000, (B,), generator=gen).numpy().astype(np.int32)
    conv_pool, ssm_pool = to_dev(cp, dev, BF16), to_dev(ssm, dev)
    dcw, dA, ddt, dslots = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(slots, dev)
    ocp, ossm = C.to_bf16_bits(cp), ssm.copy()
    cwb = C.to_bf16_bits(cw).reshape(-1)
    worst = 0.0
    for step in range(steps):
        proj = rand_bf(gen, (B, PW))
        y = qt.batch.deltanet_b(to_dev(proj, dev, BF16), conv_pool, dcw, dA, ddt, ssm_pool, dslots, to_dev(pos, dev))
        oy = C.from_bf16_bits(C.decode_step(C.to_bf16_bits(proj), ocp, cwb, A_log, dtb, ossm, slots, pos, acc64=True, nthreads=8))
        if step in state_at:
            got = to_np(ssm_pool)
            for b in range(B):
                e = rel_max(got[slots[b]], ossm[slots[b]])
                worst = max(worst, e)
                if not e <= 1e-4:
                    raise AssertionError(f"step {step}, row {b}: state relative error {e:.3e} > 1e-4")
        check_ulp(f"y at step {step}", to_np(y), oy)
        if step % 50 == 0 or step == steps - 1:
            check_equal(f"conv pool at step {step}", to_np(conv_pool), C.from_bf16_bits(ocp))
        pos = pos + 1
    check_equal("trash slot", to_np(ssm_pool[B]), ssm[B])
    print(f"1000 steps at B={B}: worst state error {worst:.2e}")


def test_deltanet_bm_config4_size(qt, dev):
    """benchmark config 4's GatedDeltaNet half at its stated size: B = 16 sequences x M = 4 draft tokens, every snapshot
    against the oracle (reference call: qwen35/batch_spec.py:142-150)."""
    rng = np.random.default_rng(1004)
    cw, A_log, dtb, gw = layer_params(12)
    NS, B, M = 16, 16, 4
    sslots = rng.permutation(NS).astype(np.int32)[:B]
    sels = rng.integers(0, M, B).astype(np.int32)
    pars = rng.integers(0, 2, B).astype(np.int32)
    cp = bf(rng.standard_normal(((NS + 1) * 2, M, 3, CD)))
    sp = (rng.standard_normal((NS + 1, M, 16, 128, 128)) * 0.02).astype(np.float32)
    proj = bf(rng.standard_normal((B * M, PW)))
    conv_pool, ssm_pool = to_dev(cp, dev, BF16), to_dev(sp, dev)
    y = qt.batch_spec.deltanet_bm(to_dev(proj, dev, BF16), conv_pool, to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev),
                                  ssm_pool, to_dev(sslots, dev), to_dev(sels, dev), to_dev(pars, dev), M)
    ocp, osp = cp.copy(), sp.copy()
    oy = O.deltanet_bm(proj, ocp, cw, A_log, dtb, osp, sslots, sels, pars, M)
    check_equal("conv pool", to_np(conv_pool), ocp)
    got = to_np(ssm_pool)
    for b in range(B):
        for j in range(M):
            check_rel(f"snapshot {j} of sequence {b}", got[sslots[b], j], osp[sslots[b], j], 1e-4, rel_max)
    check_ulp("y", to_np(y), oy)
    check_equal("trash entry", got[NS], sp[NS])


@pytest.mark.parametrize("B", [1, 5, 24, 32, 48, 64, 80])
def test_deltanet_b_gnorm_equals_two_launches(qt, dev, B):
    """the decode step with the gated RMSNorm fused in == deltanet_b followed by gnorm_rows (batch.py:497-499), bit for bit,
    for each workgroup shape the batch size selects (1, 2 or 4 heads per workgroup)"""
    gen = torch.Generator().manual_seed(200 + B)
    cw, A_log, dtb, gw = layer_params(20 + B)
    S = B + 2
    ssm = (torch.randn((S + 1, 16, 128, 128), generator=gen) * 0.05).numpy()
    cp = rand_bf(gen, ((S + 1) * 2, 3, CD))
    slots = torch.randperm(S, generator=gen).numpy().astype(np.int32)[:B]
    pos = torch.randint(0, 500, (B,), generator=gen).numpy().astype(np.int32)
    proj = to_dev(rand_bf(gen, (B, PW), 1.5), dev, BF16)
    dcw, dA, ddt, dgw = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev)
    c1, s1 = to_dev(cp, dev, BF16), to_dev(ssm, dev)
    y = qt.batch.deltanet_b(proj, c1, dcw, dA, ddt, s1, to_dev(slots, dev), to_dev(pos, dev))
    want = qt.batch.gnorm_rows(y, proj, dgw)
    c2, s2 = to_dev(cp, dev, BF16), to_dev(ssm, dev)
    got = qt.batch.deltanet_b_gnorm(proj, c2, dcw, dA, ddt, s2, to_dev(slots, dev), to_dev(pos, dev), dgw)
    check_tensors_equal("gated-norm output", got, want)
    check_tensors_equal("conv pool", c2, c1)
    check_tensors_equal("ssm pool", s2, s1)
    check_equal("against the oracle", to_np(got), O.gated_norm(to_np(y), to_np(proj), gw))
