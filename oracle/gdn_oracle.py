"""CPU restatement of the GatedDeltaNet + GQA-hd256 attention hot path of wang90063/Qwen-tailor.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this file: it is the checker that the
GPU kernels are compared against (tests/, __graft_entry__.smoke(), and the cpu_baseline leg of bench.py).

Every function cites the reference file:line it restates.  bf16 tensors are represented as float32 numpy
arrays whose values are bf16-exact; `BF` marks the points where the reference rounds to bf16.

Arithmetic contract shared with the HIP kernels (so that the elementwise prologue is bit-reproducible):
  * exp32(x) / log32(x): the float64 libm result rounded to float32 (a correctly rounded float32 function
    for all practical purposes); the reference uses metal::precise::exp / log, whose last-ulp behaviour is
    not available off Apple hardware.
  * sums of squares of bf16 values are exact (accumulated in float64) and then rounded to float32 once.
  * rsqrt(x) = 1 / sqrt(x) evaluated in float64 and rounded to float32 once.
  * the recurrence itself (dot products over Dk) is accumulated in `acc` precision (float64 by default);
    the kernels accumulate in float32, which is what the 1e-4 tolerance covers.

parity status (what pins each function is listed in tests/test_oracle_pins.py):
  pinned by closed forms / library routines / brute force: sigmoid_bf16, silu_bf16, softplus_bf16, conv_silu,
    l2norm_scale, gates, delta_rule_step, gated_delta_update, deltanet, deltanet_b, deltanet_bm, gated_norm,
    chunked_gdn, attn_b, sdpa_causal.
  parity unpinned (bit-level behaviour against live MLX / mlx-lm cannot be checked here: neither is installed
    and every reference test needs an Apple GPU): the last-ulp choice of exp/log/rsqrt above.
"""
from __future__ import annotations

import numpy as np

HV, DK, DV, KD, CD, PW = 16, 128, 128, 2048, 6144, 8224     # batch.py:29, kernels.py:466
H_Q, H_KV, D_ATT = 8, 2, 256                                # model.py:43-45
F32 = np.float32

INV_SCALE = F32(0.08838834764831845)                        # 128^-0.5, kernels.py:490
E2 = F32(F32(F32(1e-6) * INV_SCALE) * INV_SCALE)            # kernels.py:491  (eps * inv_scale * inv_scale)
ATT_SCALE = F32(0.0625)                                     # 256^-0.5, batch.py:177


# ------------------------------------------------------------------------------------------------
# bf16 rounding and the scalar helpers (mslib.py:7-27)
# ------------------------------------------------------------------------------------------------
def BF(x):
    """float32 -> bf16 (round to nearest even) -> float32.  (`#define BF(v)`, mslib.py:8-10)"""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    out = ((u + r) & np.uint32(0xFFFF0000)).view(np.float32)
    return np.where(np.isnan(x), x, out).astype(np.float32)


def exp32(x):
    with np.errstate(over="ignore", under="ignore"):
        return np.exp(np.asarray(x, dtype=np.float64)).astype(np.float32)


def log32(x):
    with np.errstate(divide="ignore"):
        return np.log(np.asarray(x, dtype=np.float64)).astype(np.float32)


def rsqrt32(x):
    return (1.0 / np.sqrt(np.asarray(x, dtype=np.float32).astype(np.float64))).astype(np.float32)


def log1p_mx(x):
    """mx_log1p (mslib.py:11-15): x * log(1+x) / ((1+x) - 1), or x when 1+x == 1."""
    x = np.asarray(x, dtype=np.float32)
    xp1 = (F32(1.0) + x).astype(np.float32)
    den = (xp1 - F32(1.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        r = (x * (log32(xp1) / den).astype(np.float32)).astype(np.float32)
    return np.where(xp1 == F32(1.0), x, r).astype(np.float32)


def sigmoid_bf16(x):
    """mx_sigmoid_bf16 (mslib.py:16-20): y = BF(1/BF(1+BF(exp|x|))); x<0 ? y : BF(1-y)."""
    x = np.asarray(x, dtype=np.float32)
    e = BF(exp32(np.abs(x)))
    with np.errstate(over="ignore"):
        d = BF((F32(1.0) + e).astype(np.float32))
        y = BF((F32(1.0) / d).astype(np.float32))
    return np.where(x < 0, y, BF((F32(1.0) - y).astype(np.float32))).astype(np.float32)


def silu_bf16(x):
    """mx_silu_bf16 (mslib.py:21-22): BF(x * sigmoid_bf16(x))."""
    x = np.asarray(x, dtype=np.float32)
    return BF((x * sigmoid_bf16(x)).astype(np.float32))


def softplus_bf16(x):
    """mx_softplus_bf16 (mslib.py:23-26): BF(max(x,0) + BF(log1p(BF(exp(-|x|)))))."""
    x = np.asarray(x, dtype=np.float32)
    t = BF(log1p_mx(BF(exp32(-np.abs(x)))))
    return BF((np.maximum(x, F32(0.0)) + t).astype(np.float32))


# ------------------------------------------------------------------------------------------------
# gates, q/k norm, conv  (kernels.py:476-515, gated_delta.py:16-30, prefill.py:96-134)
# ------------------------------------------------------------------------------------------------
def gates(a, b, A_log, dt_bias):
    """a, b [..., 16] bf16-exact; A_log, dt_bias [16] float32.  Returns (g float32, beta bf16-exact).
    av = BF(a + dt_bias); g = exp(-exp(A_log) * softplus_bf16(av)); beta = sigmoid_bf16(b)  (kernels.py:511-515,
    gated_delta.py:16-18,158)."""
    a = np.asarray(a, dtype=np.float32)
    av = BF((a + np.asarray(dt_bias, dtype=np.float32)).astype(np.float32))
    sp = softplus_bf16(av)
    A = exp32(np.asarray(A_log, dtype=np.float32))
    g = exp32(((-A) * sp).astype(np.float32))
    return g, sigmoid_bf16(b)


def log_decay(a, A_log, dt_bias):
    """lg = -exp(A_log) * softplus_bf16(BF(a + dt_bias)) in float32 (gdn_nax.py:84-87)."""
    av = BF((np.asarray(a, dtype=np.float32) + np.asarray(dt_bias, dtype=np.float32)).astype(np.float32))
    return ((-exp32(np.asarray(A_log, dtype=np.float32))) * softplus_bf16(av)).astype(np.float32)


def l2norm_scale(u, which):
    """u [..., 128] bf16-exact conv outputs -> normalized and scaled q or k (kernels.py:490-510):
    r = rsqrt(sum(u^2)/128 + e2); out = BF(BF(u*r) * sc), sc_q = BF(1/128), sc_k = BF(128^-0.5)."""
    u = np.asarray(u, dtype=np.float32)
    ss = (u.astype(np.float64) ** 2).sum(-1, keepdims=True).astype(np.float32)
    r = rsqrt32((ss / F32(DK)).astype(np.float32) + E2)
    sc = BF(INV_SCALE * INV_SCALE) if which == "q" else BF(INV_SCALE)
    return BF((BF((u * r).astype(np.float32)) * sc).astype(np.float32))


def normalize_qk(q, k):
    """normalize_qk (gated_delta.py:21-30) with inv_scale = 128^-0.5, eps = 1e-6, bf16 in/out."""
    return l2norm_scale(q, "q"), l2norm_scale(k, "k")


def conv_silu(win, x, cw):
    """Depthwise causal conv, kernel 4, then SiLU (kernels.py:480-484).
    win [..., 3, C] = the three previous pre-conv input rows, oldest first; x [..., C] the current row; cw [C, 4].
    u = silu_bf16(BF(((w0*c0 + w1*c1) + w2*c2) + x*c3))."""
    win = np.asarray(win, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    cw = np.asarray(cw, dtype=np.float32).reshape(-1, 4)
    s = (win[..., 0, :] * cw[:, 0]).astype(np.float32)
    s = (s + (win[..., 1, :] * cw[:, 1]).astype(np.float32)).astype(np.float32)
    s = (s + (win[..., 2, :] * cw[:, 2]).astype(np.float32)).astype(np.float32)
    s = (s + (x * cw[:, 3]).astype(np.float32)).astype(np.float32)
    return silu_bf16(BF(s))


def conv_prep(proj, conv_state, cw):
    """prefill.conv_prep (prefill.py:228-238): proj [S, 8224], conv_state [3, 6144], cw [6144*4] ->
    q, k [S,16,128] normalized + scaled, v [S,16,128], all bf16-exact."""
    proj = np.asarray(proj, dtype=np.float32)
    S = proj.shape[0]
    X = np.concatenate([np.asarray(conv_state, dtype=np.float32).reshape(3, CD), proj[:, :CD]], axis=0)   # [S+3, CD]
    win = np.stack([X[0:S], X[1:S + 1], X[2:S + 2]], axis=1)                                                # [S, 3, CD]
    u = conv_silu(win, X[3:], cw)
    q = l2norm_scale(u[:, :KD].reshape(S, HV, DK), "q")
    k = l2norm_scale(u[:, KD:2 * KD].reshape(S, HV, DK), "k")
    v = u[:, 2 * KD:].reshape(S, HV, DV)
    return q, k, v


# ------------------------------------------------------------------------------------------------
# the recurrence (gated_delta.py:75-126, kernels.py:518-530)
# ------------------------------------------------------------------------------------------------
def delta_rule_step(S, q, k, v, g, beta, acc=np.float64):
    """One token.  S [..., Dv, Dk] float32; q, k [..., Dk]; v [..., Dv]; g, beta [...].
    s = S*g; kv = s.k; delta = (v - kv)*beta; s += k*delta; y = s.q   -> (y [..., Dv] in `acc`, new S float32)."""
    S = np.asarray(S, dtype=acc)
    q, k, v = (np.asarray(t, dtype=acc) for t in (q, k, v))
    g = np.asarray(g, dtype=acc)[..., None, None]
    beta = np.asarray(beta, dtype=acc)[..., None]
    S = S * g
    kv = (S * k[..., None, :]).sum(-1)
    d = (v - kv) * beta
    S = S + d[..., None] * k[..., None, :]
    y = (S * q[..., None, :]).sum(-1)
    return y, S.astype(np.float32)


def gated_delta_update(q, k, v, a, b, A_log, dt_bias, state=None, acc=np.float64):
    """gated_delta_update (gated_delta.py:143-174).  q, k [B,T,Hk,Dk] (already normalized), v [B,T,Hv,Dv],
    a, b [B,T,Hv], state [B,Hv,Dv,Dk] float32 (zeros if None) -> (y [B,T,Hv,Dv] bf16-exact, state float32)."""
    q, k, v = (np.asarray(t, dtype=np.float32) for t in (q, k, v))
    B, T, Hk, Dk = k.shape
    Hv, Dv = v.shape[2:]
    if Dk != 128 or Dv % 8:
        raise ValueError("only the scalar-gate, Dk=128, fp32-state case is supported")
    g, beta = gates(a, b, A_log, dt_bias)
    S = np.zeros((B, Hv, Dv, Dk), np.float32) if state is None else np.asarray(state, dtype=np.float32).copy()
    rep = Hv // Hk
    y = np.zeros((B, T, Hv, Dv), np.float32)
    for t in range(T):
        qt = np.repeat(q[:, t], rep, axis=1)
        kt = np.repeat(k[:, t], rep, axis=1)
        yt, S = delta_rule_step(S, qt, kt, v[:, t], g[:, t], beta[:, t], acc)
        y[:, t] = BF(yt.astype(np.float32))
    return y, S


# ------------------------------------------------------------------------------------------------
# fused decode / verify step (kernels.py:461-567, batch.py:36-135, batch_spec.py:45-150)
# ------------------------------------------------------------------------------------------------
def _tokens(proj, win, cw, A_log, dt_bias, S, acc):
    """M chained tokens of one sequence.  proj [M, 8224]; win [3, 6144]; S [16,128,128] float32.
    Yields (y [2048] bf16-exact, window [3,6144], state [16,128,128]) after every token."""
    proj = np.asarray(proj, dtype=np.float32)
    win = np.asarray(win, dtype=np.float32).reshape(3, CD).copy()
    S = np.asarray(S, dtype=np.float32)
    for j in range(proj.shape[0]):
        x = proj[j]
        u = conv_silu(win, x[:CD], cw)
        q = l2norm_scale(u[:KD].reshape(HV, DK), "q")
        k = l2norm_scale(u[KD:2 * KD].reshape(HV, DK), "k")
        v = u[2 * KD:].reshape(HV, DV)
        g, beta = gates(x[CD + KD + HV:CD + KD + 2 * HV], x[CD + KD:CD + KD + HV], A_log, dt_bias)
        y, S = delta_rule_step(S, q, k, v, g, beta, acc)
        win = np.concatenate([win[1:], x[None, :CD]], axis=0)
        yield BF(y.astype(np.float32)).reshape(HV * DV), win.copy(), S


def deltanet(proj, conv_snap, cw, A_log, dt_bias, ssm_snap, sel, acc=np.float64):
    """kernels.deltanet (kernels.py:555-567): start from snapshot sel, M tokens, snapshot after each.
    Returns y [M,2048], cs [M,3,6144], st [M,16,128,128]."""
    M = proj.shape[0]
    sel = int(np.asarray(sel).reshape(-1)[0])
    ys, cs, st = [], [], []
    for y, w, S in _tokens(proj, np.asarray(conv_snap)[sel], cw, A_log, dt_bias, np.asarray(ssm_snap)[sel], acc):
        ys.append(y), cs.append(w), st.append(S)
    return np.stack(ys), np.stack(cs), np.stack(st)


def deltanet_b(proj, conv_pool, cw, A_log, dt_bias, ssm_pool, slots, pos, acc=np.float64):
    """batch.deltanet_b (batch.py:128-135).  Mutates ssm_pool[slot] and conv buffer (pos&1)^1; returns y [B,2048]."""
    B = proj.shape[0]
    y = np.zeros((B, HV * DV), np.float32)
    for b in range(B):
        s, par = int(slots[b]), int(pos[b]) & 1
        (yb, w, S), = _tokens(proj[b:b + 1], conv_pool[s * 2 + par], cw, A_log, dt_bias, ssm_pool[s], acc)
        y[b], conv_pool[s * 2 + (par ^ 1)], ssm_pool[s] = yb, w, S
    return y


def deltanet_bm(proj, conv_pool, cw, A_log, dt_bias, ssm_pool, sslots, sels, pars, M, acc=np.float64):
    """batch_spec.deltanet_bm (batch_spec.py:142-150).  ssm_pool [NS+1,M,16,128,128], conv_pool [(NS+1)*2,M,3,6144];
    row b*M+j of proj is token j of sequence b; reads snapshot sels[b] of buffer pars[b], writes snapshots 0..M-1 of
    the pool entry and of conv buffer pars[b]^1, in place.  Returns y [B*M, 2048]."""
    B = len(sslots)
    y = np.zeros((B * M, HV * DV), np.float32)
    for b in range(B):
        ss, sl, par = int(sslots[b]), int(sels[b]), int(pars[b]) & 1
        outs = list(_tokens(proj[b * M:(b + 1) * M], conv_pool[ss * 2 + par, sl], cw, A_log, dt_bias,
                            ssm_pool[ss, sl].copy(), acc))
        for j, (yj, w, S) in enumerate(outs):
            y[b * M + j], conv_pool[ss * 2 + (par ^ 1), j], ssm_pool[ss, j] = yj, w, S
    return y


# ------------------------------------------------------------------------------------------------
# gated RMSNorm (kernels.py:124-139, batch.py:304-343, prefill.py:137-157)
# ------------------------------------------------------------------------------------------------
def gated_norm(y, proj, gw, eps=1e-6):
    """y [R,2048] bf16-exact, z = proj[:, 6144:8192], gw [128] float32 ->
    BF( z/(1+exp(-z)) * (gw * (y * rsqrt(mean_128(y^2) + eps))) ) per head."""
    y = np.asarray(y, dtype=np.float32).reshape(-1, HV, DV)
    z = np.asarray(proj, dtype=np.float32)[:, CD:CD + HV * DV].reshape(-1, HV, DV)
    gw = np.asarray(gw, dtype=np.float32)
    ss = (y.astype(np.float64) ** 2).sum(-1, keepdims=True).astype(np.float32)
    inv = rsqrt32((ss / F32(128.0)).astype(np.float32) + F32(eps))
    n = (gw * (y * inv).astype(np.float32)).astype(np.float32)
    with np.errstate(over="ignore"):
        sig = (z / (F32(1.0) + exp32(-z)).astype(np.float32)).astype(np.float32)
    return BF((sig * n).astype(np.float32)).reshape(-1, HV * DV)


# ------------------------------------------------------------------------------------------------
# chunked (WY) form (gdn_nax.py:3-10, 80-142, 256-345), any chunk size C
# ------------------------------------------------------------------------------------------------
def chunk_matrices(q, k, lg, beta):
    """Phase A for one (chunk, head) in float64 (gdn_nax.py:80-142; fp64 statement in bench/gdn_nax_err.py:31-41).
    q, k [C,128]; lg [C] log-decay; beta [C].  Returns Tb [C,C], A [C,C], gamma [C], dec [C]."""
    q, k, lg, beta = (np.asarray(t, dtype=np.float64) for t in (q, k, lg, beta))
    C = q.shape[0]
    Lc = np.cumsum(lg)
    G = np.exp(Lc[:, None] - Lc[None, :])
    L = np.tril(beta[:, None] * G * (k @ k.T), -1)
    T = np.zeros((C, C))
    for j in range(C):                      # forward substitution, one column at a time (gdn_nax.py:130-141)
        x = np.zeros(C)
        for i in range(C):
            x[i] = (1.0 if i == j else 0.0) - L[i, :i] @ x[:i]
        T[:, j] = x
    return T * beta[None, :], np.tril(G * (q @ k.T)), np.exp(Lc), np.exp(Lc[-1] - Lc)


def chunked_gdn(q, k, v, lg, beta, S0, C=64):
    """gdn_chunked for all heads in float64 (gdn_nax.py:256-345).  q,k,v [T,16,128], lg, beta [T,16], S0 [16,128,128].
    A partial last chunk is padded with zero rows, lg = 0, beta = 0 (gdn_nax.py:81-90).  Returns (y [T,16,128], S1)."""
    q, k, v, lg, beta = (np.asarray(t, dtype=np.float64) for t in (q, k, v, lg, beta))
    T = q.shape[0]
    S = np.asarray(S0, dtype=np.float64).copy()
    y = np.zeros((T, HV, DV))
    for t0 in range(0, T, C):
        n = min(C, T - t0)
        pad = lambda x: np.concatenate([x[t0:t0 + n], np.zeros((C - n,) + x.shape[1:])], axis=0)
        qc, kc, vc, lc, bc = pad(q), pad(k), pad(v), pad(lg), pad(beta)
        for h in range(HV):
            Tb, A, gam, dec = chunk_matrices(qc[:, h], kc[:, h], lc[:, h], bc[:, h])
            P1 = kc[:, h] @ S[h].T
            P2 = qc[:, h] @ S[h].T
            Z = vc[:, h] - gam[:, None] * P1
            D = Tb @ Z
            Y = gam[:, None] * P2 + A @ D
            S[h] = gam[-1] * S[h] + (D * dec[:, None]).T @ kc[:, h]
            y[t0:t0 + n, h] = Y[:n]
    return y, S


def prefill_gdn(proj, conv_state, cw, A_log, dt_bias, S0, gw, acc=np.float64):
    """One GDN layer core over S tokens, sequential form: conv_prep -> recurrence -> gated norm, as
    prefill._linear_attn with QWEN35_GDN=ref (prefill.py:247-265).  Returns (out [S,2048] bf16-exact, y [S,2048]
    bf16-exact, new conv state [3,6144], new ssm state [16,128,128])."""
    proj = np.asarray(proj, dtype=np.float32)
    q, k, v = conv_prep(proj, conv_state, cw)
    y, S = gated_delta_update(q[None], k[None], v[None], proj[None, :, CD + KD + HV:CD + KD + 2 * HV],
                              proj[None, :, CD + KD:CD + KD + HV], A_log, dt_bias, np.asarray(S0)[None], acc)
    y = y[0].reshape(-1, HV * DV)
    tail = np.concatenate([np.asarray(conv_state, dtype=np.float32).reshape(3, CD), proj[:, :CD]], axis=0)[-3:]
    return gated_norm(y, proj, gw), y, tail, S[0]


# ------------------------------------------------------------------------------------------------
# attention (batch.py:141-237, model.py:160-167)
# ------------------------------------------------------------------------------------------------
def attn_b(q, k_new, v_new, Kp, Vp, slots, pos, M=1):
    """batch.attn_b (batch.py:230-237) in float64.  q [R,8,256]; k_new, v_new [R,2,256]; pools [S+1,2,Lmax,256];
    row r = b*M+j attends pool keys < pos[b] and the new keys of rows b*M..b*M+j; appends the new rows at pos[b]+j.
    Returns o [R,8,256] bf16-exact."""
    q = np.asarray(q, dtype=np.float64)
    R, H, D = q.shape
    KV = k_new.shape[1]
    o = np.zeros((R, H, D), np.float32)
    for r in range(R):
        b, j = divmod(r, M)
        s, p0 = int(slots[b]), int(pos[b])
        for h in range(H):
            kvh = h // (H // KV)
            K = np.concatenate([Kp[s, kvh, :p0], k_new[b * M:b * M + j + 1, kvh]], axis=0).astype(np.float64)
            V = np.concatenate([Vp[s, kvh, :p0], v_new[b * M:b * M + j + 1, kvh]], axis=0).astype(np.float64)
            sc = (K @ q[r, h]) * float(ATT_SCALE)
            w = np.exp(sc - sc.max())
            o[r, h] = BF((w @ V / w.sum()).astype(np.float32))
    for r in range(R):
        b, j = divmod(r, M)
        Kp[int(slots[b]), :, int(pos[b]) + j] = k_new[r]
        Vp[int(slots[b]), :, int(pos[b]) + j] = v_new[r]
    return o


def sdpa_causal(q, K, V, q_pos0=None):
    """Causal softmax(Q K^T * 256^-0.5) V with GQA (model.py:160-167), float64.  q [H,S,D]; K, V [KV,L,D];
    query i sits at absolute position q_pos0 + i (default L - S) and sees keys <= its position.  Returns bf16-exact."""
    q = np.asarray(q, dtype=np.float64)
    K = np.asarray(K, dtype=np.float64)
    V = np.asarray(V, dtype=np.float64)
    H, S, D = q.shape
    KV, L, _ = K.shape
    p0 = L - S if q_pos0 is None else q_pos0
    o = np.zeros((H, S, D), np.float32)
    for h in range(H):
        kvh = h // (H // KV)
        sc = (q[h] @ K[kvh].T) * float(ATT_SCALE)
        mask = np.arange(L)[None, :] <= (p0 + np.arange(S))[:, None]
        sc = np.where(mask, sc, -np.inf)
        w = np.exp(sc - sc.max(-1, keepdims=True))
        o[h] = BF((w @ V[kvh] / w.sum(-1, keepdims=True)).astype(np.float32))
    return o


# ------------------------------------------------------------------------------------------------
# state admission (batch.py:349-372): the strided in-place copy
# ------------------------------------------------------------------------------------------------
def blit(dst, src, n, d0, s0, ny=1, dstride=0, sstride=0):
    """dst.flat[d0 + y*dstride + i] = src.flat[s0 + y*sstride + i] for i < n, y < ny, in place on the numpy array `dst`
    (qwen35/batch.py:349-372, one element per thread of a (n, ny) grid)."""
    d, s = dst.reshape(-1), np.asarray(src).reshape(-1)
    for y in range(ny):
        d[d0 + y * dstride:d0 + y * dstride + n] = s[s0 + y * sstride:s0 + y * sstride + n]
    return dst


# ------------------------------------------------------------------------------------------------
# attention glue (batch.py:505-513, model.py:154-169): q / k RMSNorm, partial rotary embedding, output gate
# ------------------------------------------------------------------------------------------------
ROPE_DIM, ROPE_THETA, QKV_W = 64, 1e7, 8 * 512 + 2 * 2 * 256


def rope_freqs():
    """freq_i = float32(theta^(-2 i / dims)), i < dims / 2 (mx.fast.rope(..., traditional=False, base=1e7), model.py:163)"""
    return np.array([np.float32(ROPE_THETA ** (-2.0 * i / ROPE_DIM)) for i in range(ROPE_DIM // 2)], np.float32)


def rms_norm_rows(x, w, eps=1e-6):
    """mx.fast.rms_norm on rows of 256 (model.py:160-161): exact sum of squares, x * inv rounded to bf16, times the bf16 weight,
    rounded to bf16."""
    x = np.asarray(x, np.float32)
    ss = (x.astype(np.float64) ** 2).sum(-1, keepdims=True).astype(np.float32)
    inv = rsqrt32((ss / F32(x.shape[-1]) + F32(eps)).astype(np.float32))
    return BF((np.asarray(w, np.float32) * BF((x * inv).astype(np.float32))).astype(np.float32))


def rope_rows(x, pos):
    """Half-split rotary embedding of the first 64 of 256 features (mx.fast.rope, traditional=False): x [..., 256], pos
    broadcastable to x.shape[:-1].  Products and sums are rounded to float32 one by one, the result to bf16."""
    x = np.asarray(x, np.float32).copy()
    th = (np.asarray(pos, np.float32)[..., None] * rope_freqs()).astype(np.float32)
    c, s = np.cos(th.astype(np.float64)).astype(np.float32), np.sin(th.astype(np.float64)).astype(np.float32)
    x1, x2 = x[..., :32].copy(), x[..., 32:64].copy()
    x[..., :32] = BF(((x1 * c).astype(np.float32) - (x2 * s).astype(np.float32)).astype(np.float32))
    x[..., 32:64] = BF(((x1 * s).astype(np.float32) + (x2 * c).astype(np.float32)).astype(np.float32))
    return x


def attn_qkv_prep(qkv, q_norm, k_norm, pos, M=1, eps=1e-6):
    """qkv [R,5120] = [(q_h | gate_h) x 8 | k x 2 | v x 2] -> q [R,8,256], k [R,2,256] (normed + roped), v [R,2,256]
    (batch.py:505-512); row r = b*M + j sits at position pos[b] + j."""
    qkv = np.asarray(qkv, np.float32)
    R = qkv.shape[0]
    p = (np.repeat(np.asarray(pos), M) + np.tile(np.arange(M), R // M)).astype(np.float32)
    q = qkv[:, :4096].reshape(R, 8, 512)[:, :, :256]
    k = qkv[:, 4096:4608].reshape(R, 2, 256)
    v = qkv[:, 4608:].reshape(R, 2, 256).copy()
    return rope_rows(rms_norm_rows(q, q_norm, eps), p[:, None]), rope_rows(rms_norm_rows(k, k_norm, eps), p[:, None]), v


def attn_out_gate(o, qkv):
    """o [R,8,256] * sigmoid(gate) with gate_h = qkv[:, h*512+256 : (h+1)*512] (batch.py:513) -> [R,2048]"""
    o = np.asarray(o, np.float32).reshape(-1, 8, 256)
    gate = np.asarray(qkv, np.float32)[:, :4096].reshape(-1, 8, 512)[:, :, 256:]
    return BF((o * sigmoid_bf16(gate)).astype(np.float32)).reshape(-1, 2048)


# ------------------------------------------------------------------------------------------------
# the projections either side of the core (kernels.py:80-319, batch.py:249-301)
# ------------------------------------------------------------------------------------------------
def rms_rows(x, nw, eps=1e-6):
    """The `rms` prologue of fused_gemv / rms_rows (kernels.py:106-131, batch.py:249-294): inv = rsqrt(sum(x^2) / K + eps) with the
    sum of squares exact, then BF(nw * (x * inv)), each product rounded to float32."""
    x = np.asarray(x, np.float32)
    ss = (x.astype(np.float64) ** 2).sum(-1, keepdims=True).astype(np.float32)
    inv = rsqrt32((ss / F32(x.shape[-1]) + F32(eps)).astype(np.float32))
    return BF((np.asarray(nw, np.float32) * (x * inv).astype(np.float32)).astype(np.float32))


def fused_gemv(W, x, nw=None, eps=1e-6, res=None, swiglu=False, gnorm=None):
    """y = W @ f(x) (kernels.py:291-319): W [N,K], x [M,K] (bf16 values); prologue rms (nw) or gated norm (gnorm = (proj, gw));
    the products are accumulated in float64 here (the reference and the kernels accumulate in float32, in different orders);
    epilogue none: BF(s); add: BF(BF(s) + res) (kernels.py:161-169); swiglu: BF(silu_bf16(BF(s[2p])) * BF(s[2p+1]))
    (kernels.py:170-182)."""
    x = np.asarray(x, np.float32)
    if nw is not None:
        x = rms_rows(x, nw, eps)
    if gnorm is not None:
        x = gated_norm(x, gnorm[0], gnorm[1], eps)
    s = BF((x.astype(np.float64) @ np.asarray(W, np.float32).astype(np.float64).T).astype(np.float32))
    if res is not None:
        return BF((s + np.asarray(res, np.float32)).astype(np.float32))
    if swiglu:
        return BF((silu_bf16(s[:, 0::2]) * s[:, 1::2]).astype(np.float32))
    return s


# ------------------------------------------------------------------------------------------------
# prefix-cache checkpoints (prefix_cache.py:90-188): the segment format and the lookup rule
# ------------------------------------------------------------------------------------------------
def pc_segment(kv_pairs, a, pos):
    """The K / V segment of a checkpoint (prefix_cache.py:185): rows [a, pos) of every buffer, K and V of a layer interleaved,
    stacked to [2 * layers, 1, n_kv, pos - a, D]."""
    return np.stack([np.asarray(x)[:, :, a:pos] for k, v in kv_pairs for x in (k, v)])


def pc_restore(segments, max_len):
    """Fresh K / V buffers from a chain of segments (prefix_cache.py:139-154): buffer j = the chain's rows end to end, zero rows
    up to max_len.  Returns [(K, V)] per layer, each [1, n_kv, max_len, D]."""
    nb = segments[0].shape[0]
    bufs = []
    for j in range(nb):
        rows = np.concatenate([s[j] for s in segments], axis=2)
        pad = np.zeros(rows.shape[:2] + (max_len - rows.shape[2], rows.shape[3]), rows.dtype)
        bufs.append(np.concatenate([rows, pad], axis=2))
    return [(bufs[2 * i], bufs[2 * i + 1]) for i in range(nb // 2)]


def pc_lookup(nodes, ids, min_split=32, min_gain=32):
    """The lookup rule (prefix_cache.py:90-125) by plain loops.  nodes: [(toks, has_last)] with pos = len(toks).  Returns (index of
    the deepest checkpoint that is a prefix of ids or None, split position or 0)."""
    S = len(ids)
    best, part = None, 0
    for i, (toks, has_last) in enumerate(nodes):
        lcp = 0
        while lcp < min(len(toks), S) and toks[lcp] == ids[lcp]:
            lcp += 1
        if lcp == len(toks):
            if (len(toks) < S or has_last) and (best is None or len(toks) > len(nodes[best][0])):
                best = i
        elif lcp < S:
            part = max(part, lcp)
    base = len(nodes[best][0]) if best is not None else 0
    return best, (part if part >= min_split and part - base >= min_gain else 0)
