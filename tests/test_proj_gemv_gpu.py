"""GPU parity of the projections either side of the core (qwen35/kernels.py:291-319 fused_gemv, qwen35/batch.py:295-301
rms_rows) against the numpy restatement.  rms_rows is bit exact.  The product accumulates 1024 .. 3584 bf16 x bf16 terms in
float32 on the matrix cores (the reference accumulates them in float32 in another order, the restatement in float64), so its
bf16 outputs may differ by one rounding step: the tolerance is 1 bf16 ulp (2 after the add / swiglu epilogues, which round a
second time) plus 2e-5 of the largest output for sums that nearly cancel, and 2e-3 relative in the l2 norm."""
import ctypes

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


@pytest.mark.parametrize("M,K", [(1, 1024), (5, 1024), (64, 1024), (64, 2048), (3, 3584), (67, 520), (2, 8)])
def test_rms_rows_bit_exact(qt, dev, M, K):
    g = torch.Generator().manual_seed(M * 131 + K)
    x = rand_bf(g, (M, K), 1.7)
    nw = bf(1.0 + 0.2 * torch.randn(K, generator=g).numpy())
    got = qt.batch.rms_rows(to_dev(x, dev, BF16), to_dev(nw, dev, BF16), 1e-6)
    check_equal("rms_rows", to_np(got), O.rms_rows(x, nw, 1e-6))
    wide = qt.batch.rms_rows(to_dev(x, dev, BF16), to_dev(nw, dev, BF16), 1e-6, f32=True)
    assert wide.dtype == torch.float32 and torch.equal(wide, got.float())


def _close(name, got, want, ulps, inner=None):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    # the rounding step of the larger binade, plus an absolute term for sums that nearly cancel (float32 accumulation of K terms)
    tol = ulps * ulp_bf16(np.maximum(np.abs(got), np.abs(want))) + 2e-5 * np.abs(want).max()
    if inner is not None:        # an epilogue that rounds the product first: one rounding step of that (possibly larger) value
        tol = tol + ulp_bf16(np.abs(np.asarray(inner, np.float64)))
    bad = np.abs(got - want) > tol
    assert not bad.any(), f"{name}: {int(bad.sum())} of {bad.size} outputs beyond {ulps} bf16 ulp, worst {np.abs(got - want).max():.3g}"
    assert rel_l2(got, want) < 2e-3, f"{name}: rel l2 {rel_l2(got, want):.3g}"


# the six projections of a layer at decode time (hidden 1024, inter 3584), ragged row counts, a narrow and an odd-sized output
@pytest.mark.parametrize("M,N,K,epi", [
    (64, 8224, 1024, "none"), (64, 1024, 2048, "add"), (64, 5120, 1024, "none"), (64, 7168, 1024, "swiglu"), (64, 1024, 3584, "add"),
    (1, 8224, 1024, "none"), (5, 1024, 2048, "add"), (16, 7168, 1024, "swiglu"), (37, 264, 512, "none"), (70, 40, 512, "add"),
    (130, 1024, 1024, "none"), (3, 50, 512, "swiglu"),
    # wide outputs with K = 1024: rows in LDS from 4 to 64 rows (every count of 16-row blocks, partial blocks, feature counts
    # that leave the last workgroup partly or wholly past N); more than 64 rows keep the rows in registers
    (4, 8224, 1024, "none"), (17, 4096, 1024, "add"), (33, 7168, 1024, "swiglu"), (48, 4100, 1024, "none"), (63, 5120, 1024, "add"),
    (100, 8224, 1024, "none"), (3, 8224, 1024, "none"),
    # ... with each epilogue, and more row blocks than one pass of 64 rows
    (100, 4096, 1024, "add"), (70, 7168, 1024, "swiglu"), (200, 5120, 1024, "none")])
def test_fused_gemv_vs_oracle(qt, dev, M, N, K, epi):
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    W = rand_bf(g, (N, K), K ** -0.5)
    x = rand_bf(g, (M, K), 1.0)
    res = rand_bf(g, (M, N), 1.0) if epi == "add" else None
    got = qt.kernels.fused_gemv(to_dev(W, dev, BF16), to_dev(x, dev, BF16), res=None if res is None else to_dev(res, dev, BF16),
                                swiglu=epi == "swiglu")
    want = O.fused_gemv(W, x, res=res, swiglu=epi == "swiglu")
    assert tuple(got.shape) == want.shape
    # add: y = BF(BF(s) + res); when s and res nearly cancel, a product that rounds the other way moves y by one step of s
    _close(f"fused_gemv {epi}", to_np(got), want, 1 if epi == "none" else 2,
           inner=np.asarray(want, np.float64) - np.asarray(res, np.float64) if epi == "add" else None)


def test_fused_gemv_exact_on_small_integers(qt, dev):
    """with small-integer data every partial sum is exact in float32, whatever the order: the product must match bit for bit"""
    g = torch.Generator().manual_seed(11)
    M, N, K = 33, 96, 1024
    W = torch.randint(-3, 4, (N, K), generator=g).float().numpy()
    x = torch.randint(-2, 3, (M, K), generator=g).float().numpy()
    got = qt.kernels.fused_gemv(to_dev(W, dev, BF16), to_dev(x, dev, BF16))
    check_equal("integer product", to_np(got), O.fused_gemv(W, x))


@pytest.mark.parametrize("M,N,epi", [(33, 4112, 0), (64, 8224, 1), (16, 4096, 2), (5, 5120, 0)])
def test_wide_projection_exact_and_any_output_alignment(qt, dev, M, N, epi):
    """The kernel for wide outputs at K = 1024 (rows in LDS) on small-integer data, where every order of summation gives the
    same bits; and the same call through the C ABI with y and res 2 bytes off an 8-byte boundary (the general kernels take
    over) must give the same bits."""
    from qwen_tailor_amd import _lib as QL
    g = torch.Generator().manual_seed(M + N + epi)
    K = 1024
    W = torch.randint(-3, 4, (N, K), generator=g).float().numpy()
    x = torch.randint(-2, 3, (M, K), generator=g).float().numpy()
    res = torch.randint(-9, 10, (M, N), generator=g).float().numpy() if epi == 1 else None
    dW, dx = to_dev(W, dev, BF16), to_dev(x, dev, BF16)
    dres = None if res is None else to_dev(res, dev, BF16)
    got = qt.kernels.fused_gemv(dW, dx, res=dres, swiglu=epi == 2)
    want = O.fused_gemv(W, x, res=res, swiglu=epi == 2)
    if epi == 2:
        _close("integer swiglu", to_np(got), want, 1)            # silu of an integer is not an integer: within one rounding
    else:
        check_equal("integer product", to_np(got), want)
    NO = N // 2 if epi == 2 else N
    ybuf = torch.zeros(M * NO + 8, dtype=BF16, device=dev)
    rbuf = torch.zeros(M * N + 8, dtype=BF16, device=dev)
    if dres is not None:
        rbuf[1:1 + M * N] = dres.reshape(-1)
    QL.call("qt_fused_gemv", QL.ptr(dW), QL.ptr(dx), ctypes.c_void_p(rbuf.data_ptr() + 2) if dres is not None else None,
            ctypes.c_void_p(ybuf.data_ptr() + 2), M, N, K, epi, QL.stream())
    assert torch.equal(ybuf[1:1 + M * NO].reshape(M, NO), got), "outputs off an 8-byte boundary differ"


def test_fused_gemv_prologues_and_leading_dims(qt, dev):
    """nw = rms_rows first; gnorm = gated norm first (same bits as the stand-alone kernels, qwen35/batch.py:241-248);
    leading dimensions are flattened and restored; float32 x holding bf16 values is taken as is"""
    g = torch.Generator().manual_seed(12)
    W = to_dev(rand_bf(g, (256, 1024), 0.03), dev, BF16)
    x = to_dev(rand_bf(g, (2, 3, 1024), 1.0), dev, BF16)
    nw = to_dev(bf(1.0 + 0.1 * torch.randn(1024, generator=g).numpy()), dev, BF16)
    a = qt.kernels.fused_gemv(W, x, nw=nw)
    b = qt.kernels.fused_gemv(W, qt.batch.rms_rows(x.reshape(6, 1024), nw, f32=True))
    assert tuple(a.shape) == (2, 3, 256) and torch.equal(a.reshape(6, 256), b)
    Wo = to_dev(rand_bf(g, (128, 2048), 0.02), dev, BF16)
    y = to_dev(rand_bf(g, (4, 2048), 1.0), dev, BF16)
    proj = to_dev(rand_bf(g, (4, PW), 1.0), dev, BF16)
    gw = to_dev((1.0 + 0.1 * torch.randn(128, generator=g)).numpy().astype(np.float32), dev)
    res = to_dev(rand_bf(g, (4, 128), 1.0), dev, BF16)
    c = qt.kernels.fused_gemv(Wo, y, gnorm=(proj, gw), res=res)
    d = qt.kernels.fused_gemv(Wo, qt.batch.gnorm_rows(y, proj, gw), res=res)
    assert torch.equal(c, d)
    _close("gnorm + add", to_np(c), O.fused_gemv(to_np(Wo), to_np(y), gnorm=(to_np(proj), to_np(gw)), res=to_np(res)), 2)


def test_no_rows_is_not_an_error(qt, dev):
    W = torch.zeros((64, 1024), dtype=BF16, device=dev)
    x = torch.zeros((0, 1024), dtype=BF16, device=dev)
    assert tuple(qt.kernels.fused_gemv(W, x).shape) == (0, 64)
    assert tuple(qt.batch.rms_rows(x, torch.ones(1024, dtype=BF16, device=dev)).shape) == (0, 1024)


def test_fused_gemv_rejects_bad_arguments(qt, dev):
    W = torch.zeros((64, 1024), dtype=BF16, device=dev)
    x = torch.zeros((2, 1024), dtype=BF16, device=dev)
    with pytest.raises(ValueError):
        qt.kernels.fused_gemv(W, torch.zeros((2, 512), dtype=BF16, device=dev))
    with pytest.raises(ValueError):
        qt.kernels.fused_gemv(W, x, swiglu=True, res=torch.zeros((2, 64), dtype=BF16, device=dev))
    with pytest.raises(TypeError):
        qt.kernels.fused_gemv((W, W), x)
    with pytest.raises(RuntimeError):
        qt.kernels.fused_gemv(torch.zeros((64, 1000), dtype=BF16, device=dev), torch.zeros((2, 1000), dtype=BF16, device=dev))
    with pytest.raises(TypeError):
        qt.kernels.fused_gemv(W.cpu(), x)
