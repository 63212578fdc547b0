"""numpy restatement of what phase A of the chunked prefill hands to phase B (test infrastructure): the per-(chunk, head)
records Wn = -Tb (gamma*K), U = Tb V, Qh = Q, Kh = K^T, Am = A and the gate record (gamma, dec, gamma_C), packed in the MFMA
operand layouts the HIP kernels use.  Built from oracle.chunk_matrices (float64), so it checks both phase B and, later, phase A."""
import numpy as np

from oracle import gdn_oracle as O

C = 64


def kperm(kb, g, j):
    return 32 * kb + 16 * (j >> 2) + 4 * g + (j & 3)


def a_tiles(mat, n_mt, n_kb):
    """mat [16*n_mt, 32*n_kb] -> [n_mt, n_kb, 64 lanes, 8] with lane = 16 g + n holding mat[16 mt + n][kperm(kb, g, j)]"""
    out = np.zeros((n_mt, n_kb, 64, 8), np.float64)
    for g in range(4):
        for j in range(8):
            for kb in range(n_kb):
                out[:, kb, 16 * g:16 * g + 16, j] = mat[:, kperm(kb, g, j)].reshape(n_mt, 16)
    return out


def c_tiles(mat, n_mt):
    """mat [16*n_mt, 16] -> [n_mt, 64 lanes, 4] with lane (n, g) holding mat[16 mt + 4 g + r][n]"""
    out = np.zeros((n_mt, 64, 4), np.float64)
    for g in range(4):
        for r in range(4):
            out[:, 16 * g:16 * g + 16, r] = mat.reshape(n_mt, 16, 16)[:, 4 * g + r, :]
    return out


def chunk_records(q, k, v, lg, beta):
    """q, k, v [T,16,128]; lg, beta [T,16] -> dict of unpacked float64 matrices per (chunk, head) and the packed buffers
    ops [NC,16,28672] (float16), U [NC,16,8,4,64,4] (float16), gC [NC,16,132] (float32: gamma[64] | dec[64] | gamma_C, 0, 0, 0)."""
    T = q.shape[0]
    NC = (T + C - 1) // C
    ops = np.zeros((NC, 16, 28672), np.float16)
    U = np.zeros((NC, 16, 8, 4, 64, 4), np.float16)
    gC = np.zeros((NC, 16, 132), np.float32)
    raw = {}
    for c in range(NC):
        t0, n = c * C, min(C, T - c * C)
        pad = lambda x: np.concatenate([np.asarray(x[t0:t0 + n], dtype=np.float64), np.zeros((C - n,) + x.shape[1:])], axis=0)
        qc, kc, vc, lc, bc = pad(q), pad(k), pad(v), pad(lg), pad(beta)
        for h in range(16):
            Tb, A, gam, dec = O.chunk_matrices(qc[:, h], kc[:, h], lc[:, h], bc[:, h])
            Wn = -Tb @ (gam[:, None] * kc[:, h])
            Uu = Tb @ vc[:, h]
            Qg = qc[:, h]
            Kd = kc[:, h].T
            raw[(c, h)] = dict(Wn=Wn, U=Uu, Qh=Qg, Kh=Kd, Am=A, gC=gam[-1], gam=gam, dec=dec)
            rec = np.concatenate([a_tiles(Wn, 4, 4).ravel(), a_tiles(Qg, 4, 4).ravel(), a_tiles(Kd, 8, 2).ravel(),
                                  a_tiles(A, 4, 2).ravel()])
            ops[c, h] = rec.astype(np.float16)
            for s in range(8):
                U[c, h, s] = c_tiles(Uu[:, 16 * s:16 * s + 16], 4)
            gC[c, h, :64], gC[c, h, 64:128], gC[c, h, 128] = gam, dec, gam[-1]
    return raw, ops, U, gC
