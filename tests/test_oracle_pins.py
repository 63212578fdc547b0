"""Pins for the CPU oracle (oracle/gdn_oracle.py, oracle/gdn_oracle.c).

The reference holds no golden vectors for this path that can be evaluated without its weights and an Apple GPU, so
every oracle function is pinned by what the mathematics fixes: closed forms of the delta rule, library routines the
function reduces to (torch conv1d / rms_norm / scaled_dot_product_attention / numpy inv), an independent matrix
formulation by brute force on tiny shapes, and the structural invariants the reference's own tests assert
(M tokens == M single steps, batched == solo, chunked == sequential).
"""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from oracle import c_oracle as C

F32 = np.float32


def all_bf16():
    bits = (np.arange(65536, dtype=np.uint32) << 16)
    f = bits.view(np.float32)
    return f[np.isfinite(f)]


def bf(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).bfloat16().float().numpy()


def ulp_bf16(x):
    x = np.abs(np.asarray(x, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(x, 2.0 ** -126)))
    return 2.0 ** (e - 7)


# ---------------------------------------------------------------------------------------------- BF / scalar helpers
def test_bf_matches_torch_rounding():
    rng = np.random.default_rng(0)
    x = rng.integers(0, 2 ** 32, size=1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = x[np.isfinite(x)]
    ties = (np.arange(1, 4000, dtype=np.uint32) << 16 | 0x8000).view(np.float32) + F32(0)     # exact ties
    x = np.concatenate([x, ties, -ties, np.array([0.0, -0.0, np.inf, -np.inf, 3.3895314e38], np.float32)])
    assert np.array_equal(O.BF(x).view(np.uint32), bf(x).view(np.uint32))


def test_sigmoid_bf16_accuracy_symmetry_monotone():
    x = all_bf16()
    x = x[np.abs(x) < 80]
    s = O.sigmoid_bf16(x).astype(np.float64)
    ref = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    # three bf16 roundings of values <= 1: error stays below 2 ulp of the result's binade (and of 1 for x >= 0)
    tol = np.where(x < 0, 2.5 * ulp_bf16(ref), 2.0 ** -7)
    assert np.all(np.abs(s - ref) <= tol)
    xs = np.sort(x)
    assert np.all(np.diff(O.sigmoid_bf16(xs)) >= 0)
    neg = x[x < 0]
    # mirrored structure (mslib.py:19): sigmoid(+x) = BF(1 - sigmoid(-x))
    assert np.array_equal(O.sigmoid_bf16(-neg), O.BF(F32(1) - O.sigmoid_bf16(neg)))
    assert np.array_equal(O.BF(s.astype(np.float32)), s.astype(np.float32))


def test_sigmoid_softplus_silu_structure_vs_torch_bf16_ops():
    """torch evaluates each bf16 elementwise op in float32 and rounds its result to bf16 -- the same per-op rounding
    MLX applies (mslib.py:1-5).  The op-by-op torch graph must agree with the oracle except where torch's float32
    exp / log differ from the correctly rounded ones in the last place (a handful of the 65k inputs)."""
    x = all_bf16()
    x = x[np.abs(x) < 60]
    t = torch.from_numpy(x).bfloat16()
    one = torch.ones((), dtype=torch.bfloat16)
    y = one / (one + torch.exp(torch.abs(t)))
    sig = torch.where(t < 0, y, one - y).float().numpy()
    assert (sig != O.sigmoid_bf16(x)).sum() <= 8
    silu = (t * torch.where(t < 0, y, one - y)).float().numpy()
    assert (silu != O.silu_bf16(x)).sum() <= 8
    sp = (torch.clamp(t, min=0) + torch.log1p(torch.exp(-torch.abs(t)))).float().numpy()
    mism = sp != O.softplus_bf16(x)
    assert mism.sum() <= 16, mism.sum()


def test_softplus_silu_accuracy():
    x = all_bf16()
    x = x[np.abs(x) < 60]
    x64 = x.astype(np.float64)
    sp = O.softplus_bf16(x).astype(np.float64)
    ref = np.log1p(np.exp(-np.abs(x64))) + np.maximum(x64, 0)
    assert np.all(np.abs(sp - ref) <= 2.6 * ulp_bf16(ref) + 1e-40)
    si = O.silu_bf16(x).astype(np.float64)
    ref = x64 / (1 + np.exp(-x64))
    assert np.all(np.abs(si - ref) <= np.abs(x64) * 2.0 ** -7 + 1.5 * ulp_bf16(ref) + 1e-40)


def test_log1p_mx_is_log1p():
    x = np.concatenate([all_bf16()[(all_bf16() >= 0) & (all_bf16() <= 1)], np.array([1e-10, 1e-8, 3e-8], np.float32)])
    r = O.log1p_mx(x).astype(np.float64)
    ref = np.log1p(x.astype(np.float64))
    assert np.all(np.abs(r - ref) <= 4e-7 * np.abs(ref) + 1e-45)


# ---------------------------------------------------------------------------------------------- conv, norm, gates
def test_conv_silu_vs_torch_conv1d():
    rng = np.random.default_rng(1)
    S, Cn = 11, 6144
    x = bf(rng.standard_normal((S, Cn)))
    st = bf(rng.standard_normal((3, Cn)))
    cw = bf(rng.standard_normal((Cn, 4)) * 0.5)
    X = np.concatenate([st, x], 0)
    win = np.stack([X[0:S], X[1:S + 1], X[2:S + 2]], 1)
    got = O.conv_silu(win, x, cw).astype(np.float64)
    # model.py:128-131: conv1d over [state; x] with weight [C,4,1] (tap 3 multiplies the current token), groups = C
    ti = torch.from_numpy(X.astype(np.float64)).T[None]                       # [1, C, S+3]
    tw = torch.from_numpy(cw.astype(np.float64))[:, None, :]                  # [C, 1, 4]
    conv = torch.nn.functional.conv1d(ti, tw, groups=Cn)[0].T.numpy()         # [S, C]
    ref = conv / (1 + np.exp(-conv))
    err = np.abs(got - ref)
    # BF(conv) (1/2 ulp of conv, through silu' <= 1.1), BF(sigmoid) stages (<= 1.5 ulp of 1 times |x|), final BF
    assert np.all(err <= 0.55 * ulp_bf16(conv) * 1.1 + np.abs(conv) * 2.0 ** -7 + ulp_bf16(ref) + 1e-30)
    # a reversed tap order or an off-by-one window must fail by a wide margin
    bad = torch.nn.functional.conv1d(ti, tw.flip(-1), groups=Cn)[0].T.numpy()
    assert np.abs(got - bad / (1 + np.exp(-bad))).max() > 0.5


def test_conv_prep_layout_and_state_roll():
    rng = np.random.default_rng(2)
    S = 5
    proj = bf(rng.standard_normal((S, O.PW)))
    st = bf(rng.standard_normal((3, O.CD)))
    cw = bf(rng.standard_normal((O.CD, 4)) * 0.5)
    q, k, v = O.conv_prep(proj, st, cw)
    # token t of a multi-token call == a single-token call whose window is the previous three input rows
    X = np.concatenate([st, proj[:, :O.CD]], 0)
    for t in range(S):
        q1, k1, v1 = O.conv_prep(proj[t:t + 1], X[t:t + 3], cw)
        assert np.array_equal(q1[0], q[t]) and np.array_equal(k1[0], k[t]) and np.array_equal(v1[0], v[t])
    # v of head h, row r comes from channel 4096 + h*128 + r (kernels.py:520)
    u = O.conv_silu(X[None, 0:3], proj[0:1, :O.CD], cw)[0]
    assert np.array_equal(v[0, 3, 17], u[4096 + 3 * 128 + 17])


def test_l2norm_scale_norms_and_rms_norm_identity():
    rng = np.random.default_rng(3)
    u = bf(rng.standard_normal((64, 16, 128)) * 2)
    q, k = O.normalize_qk(u, u)
    kn = np.linalg.norm(k.astype(np.float64), axis=-1)
    qn = np.linalg.norm(q.astype(np.float64), axis=-1)
    sck = 0.08837890625                                                       # BF(128^-0.5)
    assert np.all(np.abs(kn - sck * np.sqrt(128)) < 3e-3)                     # ||k|| ~= 0.9999
    assert np.all(np.abs(qn - np.sqrt(128) / 128) < 3e-4)                     # ||q|| ~= 128^-0.5
    # gated_delta.py:27-30: inv_scale * rms_norm(x, eps * inv_scale^2) (library routine, float64)
    t = torch.from_numpy(u.astype(np.float64))
    inv = 128 ** -0.5
    kr = (inv * torch.nn.functional.rms_norm(t, (128,), eps=1e-6 * inv * inv)).numpy()
    qr = (inv * inv * torch.nn.functional.rms_norm(t, (128,), eps=1e-6 * inv * inv)).numpy()
    assert np.all(np.abs(k - kr) <= 2.1 * ulp_bf16(kr) + 1e-30)
    assert np.all(np.abs(q - qr) <= 2.1 * ulp_bf16(qr) + 1e-30)


def test_gates_closed_form():
    rng = np.random.default_rng(4)
    a = bf(rng.standard_normal((300, 16)) * 2)
    b = bf(rng.standard_normal((300, 16)) * 2)
    A_log = rng.uniform(0, 2.7, 16).astype(np.float32)
    dtb = bf(rng.standard_normal(16) * 0.1)
    g, beta = O.gates(a, b, A_log, dtb)
    x = bf(a + dtb).astype(np.float64)                                         # a + dt_bias is a bf16 add
    lg_ref = -np.exp(A_log.astype(np.float64)) * (np.log1p(np.exp(-np.abs(x))) + np.maximum(x, 0))
    lg = np.log(g.astype(np.float64))
    # exp, log1p and the sum inside softplus are each rounded to bf16: relative error of log g below ~3 * 2^-8
    assert np.all(np.abs(lg - lg_ref) <= 1.3e-2 * np.abs(lg_ref) + 1e-6)
    assert np.all((g > 0) & (g <= 1))
    assert np.all(np.abs(beta - 1 / (1 + np.exp(-b.astype(np.float64)))) <= 2.0 ** -7)
    assert np.allclose(np.log(np.maximum(g, 1e-38)), O.log_decay(a, A_log, dtb), rtol=1e-6, atol=1e-6)


# ---------------------------------------------------------------------------------------------- the recurrence
def test_delta_rule_closed_forms():
    rng = np.random.default_rng(5)
    S0 = (rng.standard_normal((16, 128, 128)) * 0.3).astype(np.float32)
    q = rng.standard_normal((16, 128))
    k = rng.standard_normal((16, 128))
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    v = rng.standard_normal((16, 128))
    one, zero = np.ones(16), np.zeros(16)
    # beta = 1, g = 1, ||k|| = 1: the delta rule writes the value: S' k = v
    y, S1 = O.delta_rule_step(S0, q, k, v, one, one)
    assert np.allclose(np.einsum("hvk,hk->hv", S1.astype(np.float64), k), v, atol=2e-6)
    # beta = 0: pure decay, y = g * S0 q
    g = rng.uniform(0.2, 1, 16)
    y, S1 = O.delta_rule_step(S0, q, k, v, g, zero)
    assert np.allclose(S1, S0 * g[:, None, None], rtol=1e-6)
    assert np.allclose(y, g[:, None] * np.einsum("hvk,hk->hv", S0.astype(np.float64), q), rtol=1e-9, atol=1e-9)
    # orthonormal keys, g = 1, zero state: S_T = sum_t beta_t v_t k_t^T
    Q, _ = np.linalg.qr(rng.standard_normal((128, 128)))
    S = np.zeros((1, 128, 128), np.float32)
    acc = np.zeros((128, 128))
    for t in range(6):
        bt = rng.uniform(0, 1, 1)
        vt = rng.standard_normal((1, 128))
        _, S = O.delta_rule_step(S, q[:1], Q[t][None], vt, np.ones(1), bt)
        acc += bt[0] * np.outer(vt[0], Q[t])
    assert np.allclose(S[0], acc, atol=3e-6)


def test_delta_rule_matrix_form_bruteforce_tiny():
    """Independent statement: S_t = g S_{t-1} (I - beta k k^T) + beta v k^T,  y_t = S_t q   (Dk = Dv = 4)."""
    rng = np.random.default_rng(6)
    S = rng.standard_normal((1, 4, 4)).astype(np.float32).astype(np.float64)
    Sm = S[0].copy()
    for t in range(7):
        q, k, v = rng.standard_normal((3, 1, 4))
        g, b = rng.uniform(0.1, 1, 1), rng.uniform(0, 1, 1)
        y, S = O.delta_rule_step(S, q, k, v, g, b)
        S = S.astype(np.float64)
        Sm = g[0] * Sm @ (np.eye(4) - b[0] * np.outer(k[0], k[0])) + b[0] * np.outer(v[0], k[0])
        assert np.allclose(Sm, S[0], atol=1e-5)
        assert np.allclose(Sm @ q[0], y[0], atol=1e-5)
        Sm = S[0].copy()


def _layer_params(rng):
    cw = bf(rng.standard_normal((O.CD, 4)) * 0.5)
    A_log = rng.uniform(0, 2.7, 16).astype(np.float32)
    dtb = bf(rng.standard_normal(16) * 0.1)
    return cw, A_log, dtb


def test_gated_delta_update_api():
    rng = np.random.default_rng(7)
    B, T = 2, 5
    q = bf(rng.standard_normal((B, T, 8, 128)))
    k = bf(rng.standard_normal((B, T, 8, 128)))
    v = bf(rng.standard_normal((B, T, 16, 128)))
    a = bf(rng.standard_normal((B, T, 16)))
    b = bf(rng.standard_normal((B, T, 16)))
    _, A_log, dtb = _layer_params(rng)
    q, k = O.normalize_qk(q, k)
    st = (rng.standard_normal((B, 16, 128, 128)) * 0.1).astype(np.float32)
    y, s = O.gated_delta_update(q, k, v, a, b, A_log, dtb, st)
    # Hk -> Hv map hk = hv // (Hv/Hk) (gated_delta.py:46): head 5 uses q/k head 2
    g, beta = O.gates(a, b, A_log, dtb)
    S = st[:, 5].copy()
    for t in range(T):
        yt, S = O.delta_rule_step(S, q[:, t, 2], k[:, t, 2], v[:, t, 5], g[:, t, 5], beta[:, t, 5])
        assert np.array_equal(O.BF(yt.astype(np.float32)), y[:, t, 5])
    assert np.array_equal(S, s[:, 5])
    # state=None -> zeros (gated_delta.py:162-163); T tokens == T chained calls (state carried)
    y0, s0 = O.gated_delta_update(q, k, v, a, b, A_log, dtb)
    yz, sz = O.gated_delta_update(q, k, v, a, b, A_log, dtb, np.zeros_like(st))
    assert np.array_equal(y0, yz) and np.array_equal(s0, sz)
    sc = st
    for t in range(T):
        yt, sc = O.gated_delta_update(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], a[:, t:t + 1], b[:, t:t + 1], A_log, dtb, sc)
        assert np.array_equal(yt[:, 0], y[:, t])
    assert np.array_equal(sc, s)
    with pytest.raises(ValueError):                                             # gated_delta.py:164-166
        O.gated_delta_update(q[..., :64], k[..., :64], v[..., :64], a, b, A_log, dtb)


# ---------------------------------------------------------------------------------------------- fused step, pools
def test_deltanet_m_tokens_equal_single_steps_and_sel():
    rng = np.random.default_rng(8)
    cw, A_log, dtb = _layer_params(rng)
    M = 3
    proj = bf(rng.standard_normal((M, O.PW)) * 1.5)
    cs = bf(rng.standard_normal((4, 3, O.CD)))
    ss = (rng.standard_normal((4, 16, 128, 128)) * 0.1).astype(np.float32)
    y, c, s = O.deltanet(proj, cs, cw, A_log, dtb, ss, np.array([2]))
    c1, s1 = cs[2:3], ss[2:3]
    for j in range(M):                                                          # tests/verify.py:28-33
        yj, c1, s1 = O.deltanet(proj[j:j + 1], c1, cw, A_log, dtb, s1, np.array([0]))
        assert np.array_equal(yj[0], y[j]) and np.array_equal(c1[0], c[j]) and np.array_equal(s1[0], s[j])
    # conv snapshot j = the last three input rows after token j (kernels.py:531)
    X = np.concatenate([cs[2], proj[:, :O.CD]], 0)
    for j in range(M):
        assert np.array_equal(c[j], X[j + 1:j + 4])
    # equals conv_prep + recurrence + (no norm) assembled from the separate pieces
    q, k, v = O.conv_prep(proj, cs[2], cw)
    yy, sf = O.gated_delta_update(q[None], k[None], v[None], proj[None, :, 8208:8224], proj[None, :, 8192:8208], A_log, dtb, ss[2:3])
    assert np.array_equal(yy[0].reshape(M, 2048), y) and np.array_equal(sf[0], s[-1])


def test_deltanet_b_equals_solo_and_pool_conventions():
    rng = np.random.default_rng(11)                                             # layout of tests/batch.py:42-71
    cw, A_log, dtb = _layer_params(rng)
    S, B = 6, 5
    slots = np.array([3, 0, 5, 1, 2], np.int32)
    pos = np.array([0, 1, 7, 100, 2047], np.int32)
    proj = bf(rng.standard_normal((B, O.PW)) * 2)
    cv = bf(rng.standard_normal((S + 1, 3, O.CD)))
    ssm0 = (rng.standard_normal((S + 1, 16, 128, 128)) * 0.3).astype(np.float32)
    cp = np.zeros(((S + 1) * 2, 3, O.CD), np.float32)
    for b in range(B):
        cp[slots[b] * 2 + (pos[b] & 1)] = cv[slots[b]]
    cp0, ssm = cp.copy(), ssm0.copy()
    y = O.deltanet_b(proj, cp, cw, A_log, dtb, ssm, slots, pos)
    for b in range(B):
        s_ = int(slots[b])
        ry, rc, rs = O.deltanet(proj[b:b + 1], cv[s_:s_ + 1], cw, A_log, dtb, ssm0[s_:s_ + 1], np.array([0]))
        assert np.array_equal(y[b], ry[0]) and np.array_equal(ssm[s_], rs[0])
        assert np.array_equal(cp[s_ * 2 + ((pos[b] & 1) ^ 1)], rc[0])
        assert np.array_equal(cp[s_ * 2 + (pos[b] & 1)], cp0[s_ * 2 + (pos[b] & 1)])
    assert np.array_equal(ssm[4], ssm0[4]) and np.array_equal(ssm[6], ssm0[6])


def test_deltanet_bm_equals_solo():
    rng = np.random.default_rng(0)                                              # layout of tests/batch_spec.py:40-67
    cw, A_log, dtb = _layer_params(rng)
    NS, B, M = 6, 4, 3
    sslots = np.array([4, 1, 5, 0], np.int32)
    sels = np.array([2, 0, 1, 2], np.int32)
    pars = np.array([1, 0, 0, 1], np.int32)
    cp = bf(rng.standard_normal(((NS + 1) * 2, M, 3, O.CD)))
    sp = (rng.standard_normal((NS + 1, M, 16, 128, 128)) * 0.1).astype(np.float32)
    proj = bf(rng.standard_normal((B * M, O.PW)) * 1.5)
    cp0, sp0 = cp.copy(), sp.copy()
    y = O.deltanet_bm(proj, cp, cw, A_log, dtb, sp, sslots, sels, pars, M)
    for b in range(B):
        s_, sl, pr = int(sslots[b]), int(sels[b]), int(pars[b])
        yr, cr, sr = O.deltanet(proj[b * M:(b + 1) * M], cp0[s_ * 2 + pr], cw, A_log, dtb, sp0[s_], np.array([sl]))
        assert np.array_equal(y[b * M:(b + 1) * M], yr) and np.array_equal(cp[s_ * 2 + (pr ^ 1)], cr)
        assert np.array_equal(sp[s_], sr) and np.array_equal(cp[s_ * 2 + pr], cp0[s_ * 2 + pr])
    for e in (2, 3, 6):
        assert np.array_equal(sp[e], sp0[e]) and np.array_equal(cp[2 * e], cp0[2 * e])


def test_c_oracle_matches_numpy_oracle():
    rng = np.random.default_rng(12)
    cw, A_log, dtb = _layer_params(rng)
    S, B = 4, 4
    slots = np.array([2, 0, 3, 1], np.int32)
    pos = np.array([0, 5, 8, 11], np.int32)
    proj = bf(rng.standard_normal((B, O.PW)) * 2)
    cp = bf(rng.standard_normal(((S + 1) * 2, 3, O.CD)))
    ssm = (rng.standard_normal((S + 1, 16, 128, 128)) * 0.1).astype(np.float32)
    cp_c, ssm_c = C.to_bf16_bits(cp), ssm.copy()
    y = O.deltanet_b(proj, cp, cw, A_log, dtb, ssm, slots, pos)
    yc = C.decode_step(C.to_bf16_bits(proj), cp_c, C.to_bf16_bits(cw).reshape(-1), A_log, dtb, ssm_c, slots, pos,
                       acc64=True, nthreads=2)
    assert np.array_equal(C.from_bf16_bits(cp_c), cp)                           # conv windows: bit exact
    assert np.abs(ssm_c - ssm).max() <= 1e-6 * np.abs(ssm).max()                # fp64 sums, different order
    d = np.abs(C.from_bf16_bits(yc) - y)
    assert np.all(d <= ulp_bf16(y) + 1e-30) and (d > 0).mean() < 1e-3
    # float accumulation (the timed CPU baseline) stays within the decode tolerance
    ssm_f, cp_f = ssm_c.copy(), cp_c.copy()
    C.decode_step(C.to_bf16_bits(proj), cp_f, C.to_bf16_bits(cw).reshape(-1), A_log, dtb, ssm_f, slots, pos ^ 1,
                  acc64=False, nthreads=2)
    ssm_d, cp_d = ssm_c.copy(), cp_c.copy()
    C.decode_step(C.to_bf16_bits(proj), cp_d, C.to_bf16_bits(cw).reshape(-1), A_log, dtb, ssm_d, slots, pos ^ 1,
                  acc64=True, nthreads=1)
    assert np.linalg.norm(ssm_f - ssm_d) <= 1e-5 * np.linalg.norm(ssm_d)
    # sequential kernel
    q, k, v = (bf(rng.standard_normal((1, 6, 16, 128))) for _ in range(3))
    q, k = O.normalize_qk(q, k)
    a, b = bf(rng.standard_normal((2, 1, 6, 16)))
    g, beta = O.gates(a, b, A_log, dtb)
    st = (rng.standard_normal((1, 16, 128, 128)) * 0.1).astype(np.float32)
    yr, sr = O.gated_delta_update(q, k, v, a, b, A_log, dtb, st)
    st_c = st.copy()
    yc = C.recurrent(C.to_bf16_bits(q), C.to_bf16_bits(k), C.to_bf16_bits(v), g, C.to_bf16_bits(beta), st_c, True, 2)
    assert np.abs(st_c - sr).max() <= 2e-6 * np.abs(sr).max()
    assert np.all(np.abs(C.from_bf16_bits(yc) - yr) <= ulp_bf16(yr) + 1e-30)


# ---------------------------------------------------------------------------------------------- gated norm
def test_gated_norm_vs_torch_rms_norm():
    rng = np.random.default_rng(13)
    y = bf(rng.standard_normal((7, 2048)) * 3)
    proj = bf(rng.standard_normal((7, O.PW)) * 2)
    gw = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    got = O.gated_norm(y, proj, gw)
    ty = torch.from_numpy(y.astype(np.float64)).reshape(7, 16, 128)
    tz = torch.from_numpy(proj[:, 6144:8192].astype(np.float64)).reshape(7, 16, 128)
    ref = (torch.nn.functional.rms_norm(ty, (128,), torch.from_numpy(gw.astype(np.float64)), 1e-6)
           * torch.nn.functional.silu(tz)).reshape(7, 2048).numpy()               # model.py:137-139
    assert np.all(np.abs(got - ref) <= 0.51 * ulp_bf16(ref) + 1e-6 * np.abs(ref) + 1e-30)


# ---------------------------------------------------------------------------------------------- chunked form
def test_chunk_inverse_vs_numpy_inv():
    rng = np.random.default_rng(14)
    C_ = 64
    q, k = rng.standard_normal((2, C_, 128)) / np.sqrt(128)
    k[5] = k[4]                                                                  # correlated keys (gdn_nax.py:118-119)
    lg = -rng.uniform(0, 0.3, C_)
    beta = rng.uniform(0, 1, C_)
    Tb, A, gam, dec = O.chunk_matrices(q, k, lg, beta)
    Lc = np.cumsum(lg)
    G = np.exp(Lc[:, None] - Lc[None, :])
    Lm = np.tril(beta[:, None] * G * (k @ k.T), -1)
    assert np.allclose(Tb, np.linalg.inv(np.eye(C_) + Lm) * beta[None, :], atol=1e-12)   # bench/gdn_nax_err.py:38-39
    assert np.allclose(A, np.tril(G * (q @ k.T)), atol=1e-14)
    assert np.allclose(gam, np.exp(Lc)) and np.allclose(dec, np.exp(Lc[-1] - Lc))


@pytest.mark.parametrize("T,C_", [(5, 64), (16, 16), (37, 16), (130, 64), (64, 1), (70, 64)])
def test_chunked_equals_sequential(T, C_):
    rng = np.random.default_rng(15)
    q, k, v = rng.standard_normal((3, T, 16, 128))
    q /= np.linalg.norm(q, axis=-1, keepdims=True) * np.sqrt(128)
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    lg = -rng.uniform(0, 0.5, (T, 16))
    beta = rng.uniform(0, 1, (T, 16))
    S0 = rng.standard_normal((16, 128, 128)) * 0.02
    yc, Sc = O.chunked_gdn(q, k, v, lg, beta, S0, C=C_)
    S = S0.copy()
    ys = np.zeros_like(yc)
    for t in range(T):                                                           # float64 state, no fp32 storage rounding
        S = S * np.exp(lg[t])[:, None, None]
        kv = np.einsum("hvk,hk->hv", S, k[t])
        d = (v[t] - kv) * beta[t][:, None]
        S = S + d[:, :, None] * k[t][:, None, :]
        ys[t] = np.einsum("hvk,hk->hv", S, q[t])
    assert np.abs(yc - ys).max() <= 1e-11 and np.abs(Sc - S).max() <= 1e-11


# ---------------------------------------------------------------------------------------------- attention
def test_attn_b_vs_torch_sdpa_and_append():
    rng = np.random.default_rng(16)
    S, Lmax, B, M = 3, 80, 3, 3
    Kp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    Vp = bf(rng.standard_normal((S + 1, 2, Lmax, 256)))
    K0, V0 = Kp.copy(), Vp.copy()
    slots = np.array([2, 0, 1], np.int32)
    pos = np.array([0, 1, 70], np.int32)
    q = bf(rng.standard_normal((B * M, 8, 256)))
    kn = bf(rng.standard_normal((B * M, 2, 256)))
    vn = bf(rng.standard_normal((B * M, 2, 256)))
    o = O.attn_b(q, kn, vn, Kp, Vp, slots, pos, M)
    for b in range(B):                                                           # tests/batch_spec.py:82-98
        s_, p = int(slots[b]), int(pos[b])
        K1, V1 = K0[s_].copy(), V0[s_].copy()
        K1[:, p:p + M] = kn[b * M:(b + 1) * M].transpose(1, 0, 2)
        V1[:, p:p + M] = vn[b * M:(b + 1) * M].transpose(1, 0, 2)
        L = p + M
        tq = torch.from_numpy(q[b * M:(b + 1) * M].transpose(1, 0, 2).astype(np.float64))[None]
        tk = torch.from_numpy(K1[:, :L].astype(np.float64)).repeat_interleave(4, 0)[None]
        tv = torch.from_numpy(V1[:, :L].astype(np.float64)).repeat_interleave(4, 0)[None]
        mask = torch.arange(L)[None, :] <= (p + torch.arange(M))[:, None]
        r = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask, scale=256 ** -0.5)[0]
        r = r.permute(1, 0, 2).numpy()
        assert np.all(np.abs(o[b * M:(b + 1) * M] - r) <= 0.51 * ulp_bf16(r) + 1e-9)
        assert np.array_equal(Kp[s_, :, p:p + M], kn[b * M:(b + 1) * M].transpose(1, 0, 2))
        assert np.array_equal(Vp[s_, :, p:p + M], vn[b * M:(b + 1) * M].transpose(1, 0, 2))
        assert np.array_equal(Kp[s_, :, :p], K0[s_, :, :p]) and np.array_equal(Kp[s_, :, p + M:], K0[s_, :, p + M:])
    assert np.array_equal(Kp[3], K0[3])
    # a single key: o = v
    o1 = O.attn_b(q[:1], kn[:1], vn[:1], Kp, Vp, np.array([3]), np.array([0]), 1)
    assert np.array_equal(o1[0, :4], np.broadcast_to(vn[0, 0], (4, 256))) and np.array_equal(o1[0, 4:], np.broadcast_to(vn[0, 1], (4, 256)))


def test_sdpa_causal_vs_torch():
    rng = np.random.default_rng(17)
    S = 37
    q = bf(rng.standard_normal((8, S, 256)))
    K = bf(rng.standard_normal((2, S, 256)))
    V = bf(rng.standard_normal((2, S, 256)))
    o = O.sdpa_causal(q, K, V)
    r = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q.astype(np.float64))[None], torch.from_numpy(K.astype(np.float64)).repeat_interleave(4, 0)[None],
        torch.from_numpy(V.astype(np.float64)).repeat_interleave(4, 0)[None], is_causal=True, scale=256 ** -0.5)[0].numpy()
    assert np.all(np.abs(o - r) <= 0.51 * ulp_bf16(r) + 1e-9)


# ------------------------------------------------------------------------------------------------
# attention glue and the state copy: library routines, closed forms, invariants
# ------------------------------------------------------------------------------------------------
def test_rms_norm_rows_vs_torch():
    """the q / k RMSNorm reduces to torch.nn.functional.rms_norm in float64, up to its two bf16 roundings"""
    rng = np.random.default_rng(0)
    x = bf(rng.standard_normal((5, 8, 256)) * 3)
    w = bf(1 + 0.2 * rng.standard_normal(256))
    got = O.rms_norm_rows(x, w, 1e-6)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (256,), torch.from_numpy(w).double(), 1e-6).numpy()
    assert np.all(np.abs(got - ref) <= 2.0 * ulp_bf16(ref) + 1e-30)             # two bf16 roundings (of x * inv, then of w * that)
    one = O.rms_norm_rows(np.full((1, 256), 2.0, np.float32), np.ones(256, np.float32), 0.0)
    assert np.array_equal(one, np.ones((1, 256), np.float32))                   # constant row: x / |x|


def test_rope_rows_closed_forms():
    rng = np.random.default_rng(1)
    x = bf(rng.standard_normal((7, 2, 256)))
    f = O.rope_freqs()
    assert f[0] == 1.0 and abs(float(f[16]) - 1e7 ** -0.5) < 1e-9 and np.all(np.diff(f) < 0)      # theta^(-2i/64)
    assert np.array_equal(O.rope_rows(x, np.zeros((7, 1))), x)                                    # position 0: identity
    y = O.rope_rows(x, np.arange(7, dtype=np.float32)[:, None] * 100 + 3)
    assert np.array_equal(y[..., 64:], x[..., 64:])                                               # features >= 64 pass through
    n0 = x[..., :32] ** 2 + x[..., 32:64] ** 2                                                    # a rotation keeps the pair norms
    n1 = y[..., :32] ** 2 + y[..., 32:64] ** 2
    assert np.abs(n1 - n0).max() <= 0.02 * n0.max()
    # pairing is (i, i + 32): a unit vector on feature i at position p lands on (cos, sin)(p * f_i) of features i, i + 32
    e = np.zeros((1, 256), np.float32)
    e[0, 5] = 1.0
    r = O.rope_rows(e, np.array([[11.0]]))[0]
    assert abs(r[5] - np.cos(11 * float(f[5]))) < 4e-3 and abs(r[37] - np.sin(11 * float(f[5]))) < 4e-3 and np.count_nonzero(r) == 2
    # relative-position property: <rope(q, p), rope(k, p')> depends on p - p' only (float64 check of the formula, no rounding)
    q, k = rng.standard_normal(256), rng.standard_normal(256)
    def rot(v, p):
        v = v.copy()
        c, s = np.cos(p * f.astype(np.float64)), np.sin(p * f.astype(np.float64))
        v[:32], v[32:64] = v[:32] * c - v[32:64] * s, v[:32] * s + v[32:64] * c
        return v
    assert abs(rot(q, 17.0) @ rot(k, 5.0) - rot(q, 112.0) @ rot(k, 100.0)) < 1e-9


def test_attn_qkv_prep_and_gate_layout():
    rng = np.random.default_rng(2)
    R, M = 6, 2
    qkv = bf(rng.standard_normal((R, O.QKV_W)))
    qn, kn = bf(1 + 0.1 * rng.standard_normal(256)), bf(1 + 0.1 * rng.standard_normal(256))
    pos = np.array([4, 0, 1000], np.int32)
    q, k, v = O.attn_qkv_prep(qkv, qn, kn, pos, M)
    assert q.shape == (R, 8, 256) and k.shape == (R, 2, 256) and v.shape == (R, 2, 256)
    assert np.array_equal(v, qkv[:, 4608:].reshape(R, 2, 256))
    # row 2 = sequence 1, token 0, position 0: no rotation, only the norm; head 3 reads columns 3*512 .. 3*512+255
    assert np.array_equal(q[2, 3], O.rms_norm_rows(qkv[2, 3 * 512:3 * 512 + 256][None], qn)[0])
    assert np.array_equal(k[2, 1], O.rms_norm_rows(qkv[2, 4096 + 256:4096 + 512][None], kn)[0])
    # row 1 = sequence 0, token 1 sits at position 5
    assert np.array_equal(q[1, 0], O.rope_rows(O.rms_norm_rows(qkv[1, :256][None], qn), np.array([[5.0]]))[0])
    o = bf(rng.standard_normal((R, 8, 256)))
    g = O.attn_out_gate(o, qkv)
    ref = o.astype(np.float64) / (1 + np.exp(-qkv[:, :4096].reshape(R, 8, 512)[:, :, 256:].astype(np.float64)))
    assert np.abs(g.reshape(R, 8, 256) - ref).max() <= 0.02 * np.abs(ref).max()


def test_blit_is_a_strided_copy():
    rng = np.random.default_rng(3)
    dst, src = rng.standard_normal(400).astype(np.float32), rng.standard_normal(300).astype(np.float32)
    d0 = dst.copy()
    O.blit(dst, src, 10, 7, 3, ny=3, dstride=100, sstride=50)
    want = d0.copy()
    for y in range(3):
        for i in range(10):
            want[7 + y * 100 + i] = src[3 + y * 50 + i]
    assert np.array_equal(dst, want)


# ------------------------------------------------------------------------------------------------
# the projections either side of the core
# ------------------------------------------------------------------------------------------------
def test_rms_rows_vs_torch_and_constant_row():
    """the rms prologue reduces to torch's rms_norm in float64 up to its single bf16 rounding; a constant row maps to the weight"""
    rng = np.random.default_rng(5)
    x = bf(rng.standard_normal((7, 1024)) * 2)
    w = bf(1 + 0.3 * rng.standard_normal(1024))
    got = O.rms_rows(x, w, 1e-6)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (1024,), torch.from_numpy(w).double(), 1e-6).numpy()
    assert np.all(np.abs(got - ref) <= 0.502 * ulp_bf16(ref) + 1e-30)           # one rounding (plus float32 products)
    assert np.array_equal(O.rms_rows(np.full((1, 512), -4.0, np.float32), w[:512], 0.0), -w[None, :512])


def test_fused_gemv_bruteforce_and_epilogues():
    """the product by plain loops on a tiny case with small-integer data (every partial sum exact, so no accumulation order
    matters); the epilogues by their closed forms; the prologues compose with the product"""
    rng = np.random.default_rng(6)
    M, N, K = 3, 6, 16
    W = rng.integers(-4, 5, (N, K)).astype(np.float32)
    x = rng.integers(-3, 4, (M, K)).astype(np.float32)
    want = np.zeros((M, N), np.float32)
    for m in range(M):
        for n in range(N):
            s = 0.0
            for k in range(K):
                s += float(W[n, k]) * float(x[m, k])
            want[m, n] = s
    assert np.array_equal(O.fused_gemv(W, x), want)                              # |s| <= 192: every sum is a bf16 value
    res = bf(rng.standard_normal((M, N)))
    assert np.array_equal(O.fused_gemv(W, x, res=res), bf(bf(want) + res))
    sw = O.fused_gemv(W, x, swiglu=True)
    g, u = bf(want[:, 0::2]), bf(want[:, 1::2])
    assert sw.shape == (M, N // 2) and np.array_equal(sw, bf(O.silu_bf16(g) * u))
    # linearity in W where every value stays exactly representable
    assert np.array_equal(O.fused_gemv(2 * W, x), 2 * O.fused_gemv(W, x))
    # the rms prologue is applied to x before the product
    nw = bf(1 + 0.1 * rng.standard_normal(K))
    xr = bf(rng.standard_normal((M, K)))
    assert np.array_equal(O.fused_gemv(W, xr, nw=nw), O.fused_gemv(W, O.rms_rows(xr, nw)))
    # rounding: a product that needs more than 8 bits rounds to nearest even
    assert O.fused_gemv(np.array([[257.0]], np.float32), np.array([[1.0]], np.float32))[0, 0] == 256.0
    assert O.fused_gemv(np.array([[259.0]], np.float32), np.array([[1.0]], np.float32))[0, 0] == 260.0


def test_fused_gemv_gnorm_prologue_is_gated_norm():
    rng = np.random.default_rng(8)
    y = bf(rng.standard_normal((2, 2048)))
    proj = bf(rng.standard_normal((2, O.PW)))
    gw = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    W = bf(rng.standard_normal((8, 2048)) * 0.05)
    assert np.array_equal(O.fused_gemv(W, y, gnorm=(proj, gw)), O.fused_gemv(W, O.gated_norm(y, proj, gw)))


# ---------------------------------------------------------------------------------------------- the layer core as a whole
def _layer_core_float64(proj, cs, cw, A_log, dtb, S0, gw, swap_gates=False):
    """An independent composition of the GatedDeltaNet layer core in float64, with no bf16 rounding anywhere and none of the
    oracle's helpers: torch.conv1d over [state; x] (model.py:128-131), SiLU, textbook L2 normalisation of q and k
    (gated_delta.py:21-30), textbook gates (gated_delta.py:16-18,158), the matrix form of the delta rule per head
    S_t = g S (I - beta k k^T) + beta v k^T, y_t = S_t q, and rms_norm(y) * silu(z) (model.py:137-139)."""
    T = proj.shape[0]
    X = np.concatenate([cs, proj[:, :6144]], 0).astype(np.float64)
    conv = torch.nn.functional.conv1d(torch.from_numpy(X).T[None], torch.from_numpy(cw.astype(np.float64))[:, None, :], groups=6144)[0].T
    u = torch.nn.functional.silu(conv).numpy()
    q, k, v = (u[:, i * 2048:(i + 1) * 2048].reshape(T, 16, 128) for i in range(3))
    k = k / np.linalg.norm(k, axis=-1, keepdims=True)
    q = q / np.linalg.norm(q, axis=-1, keepdims=True) / np.sqrt(128.0)
    z = proj[:, 6144:8192].astype(np.float64).reshape(T, 16, 128)
    b_in, a_in = proj[:, 8192:8208].astype(np.float64), proj[:, 8208:8224].astype(np.float64)
    if swap_gates:
        a_in, b_in = b_in, a_in
    g = np.exp(-np.exp(A_log.astype(np.float64)) * np.logaddexp(0.0, a_in + dtb.astype(np.float64)))
    beta = 1.0 / (1.0 + np.exp(-b_in))
    S = S0.astype(np.float64).copy()                                             # [head][dv][dk]
    y = np.zeros((T, 16, 128))
    for t in range(T):
        for h in range(16):
            kk = k[t, h]
            S[h] = g[t, h] * S[h] @ (np.eye(128) - beta[t, h] * np.outer(kk, kk)) + beta[t, h] * np.outer(v[t, h], kk)
            y[t, h] = S[h] @ q[t, h]
    out = (torch.nn.functional.rms_norm(torch.from_numpy(y), (128,), torch.from_numpy(gw.astype(np.float64)), 1e-6)
           * torch.nn.functional.silu(torch.from_numpy(z))).reshape(T, 2048).numpy()
    return out, y.reshape(T, 2048), S


@pytest.mark.parametrize("T", [1, 2, 8])
def test_prefill_gdn_vs_independent_float64_composition(T):
    """O.prefill_gdn (the composition the chunked-prefill GPU tests compare with) against a composition that shares nothing with
    it: column layout of the projection row, head mapping, state layout [dv][dk], conv tail.  The two differ by the bf16
    roundings of the reference's arithmetic only (a few 2^-8 steps per stage); a swapped gate column, a transposed state or a
    shifted conv window differ by tens of percent."""
    rng = np.random.default_rng(40 + T)
    cw, A_log, dtb = _layer_params(rng)
    gw = rng.uniform(0.5, 1.5, 128).astype(np.float32)
    proj = bf(rng.standard_normal((T, O.PW)))
    cs = bf(rng.standard_normal((3, O.CD)))
    S0 = (rng.standard_normal((16, 128, 128)) * 0.5).astype(np.float32)
    out, y, tail, S1 = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    rout, ry, rS = _layer_core_float64(proj, cs, cw, A_log, dtb, S0, gw)
    rel = lambda a, b: float(np.linalg.norm(np.asarray(a, np.float64) - b) / np.linalg.norm(b))
    assert rel(S1, rS) < 1e-2                  # k, v, beta each carry a bf16 rounding (2^-9) into every rank-one term
    assert rel(y, ry) < 2e-2
    assert rel(out, rout) < 2.5e-2
    assert np.array_equal(tail, np.concatenate([cs, proj[:, :6144]], 0)[-3:])       # prefill.py:262-263
    # plausible mistakes are far outside those bounds
    bout, by, bS = _layer_core_float64(proj, cs, cw, A_log, dtb, S0, gw, swap_gates=True)
    assert rel(y, by) > 0.1
    ty = _layer_core_float64(proj, cs, cw, A_log, dtb, np.ascontiguousarray(S0.transpose(0, 2, 1)), gw)[1]
    assert rel(y[0], ty[0]) > 0.1                                                 # (the first token reads the initial state undecayed)
    sy = _layer_core_float64(proj, np.roll(cs, 1, axis=0), cw, A_log, dtb, S0, gw)[1]
    assert rel(y, sy) > 0.1
