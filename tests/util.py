"""Shared helpers of the parity tests: seeded inputs in the shapes of the benchmark configs, bf16 <-> numpy conversions
and the error measures the tolerances are written in."""
import numpy as np
import torch

HV, DK, DV, KD, CD, PW = 16, 128, 128, 2048, 6144, 8224
BF16 = torch.bfloat16


def to_np(t):
    """torch tensor (any device; bf16 -> exact float32) -> numpy"""
    t = t.detach().cpu()
    return (t.float() if t.dtype == BF16 else t).numpy()


def to_dev(x, dev, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(dev)


def bf(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).bfloat16().float().numpy()


def ulp_bf16(x):
    x = np.abs(np.asarray(x, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(x, 2.0 ** -126)))
    return 2.0 ** (e - 7)


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def rel_max(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-300))


def layer_params(seed):
    """conv_w [6144,4] bf16-exact, A_log ~ U[0,2.7], dt_bias ~ N(0,0.1) (bf16-exact), gnorm weight float32 [128]"""
    g = torch.Generator().manual_seed(seed)
    cw = (torch.randn((CD, 4), generator=g) * 0.5).bfloat16().float().numpy()
    A_log = (torch.rand(HV, generator=g) * 2.7).numpy().astype(np.float32)
    dtb = (torch.randn(HV, generator=g) * 0.1).bfloat16().float().numpy()
    gw = (1.0 + 0.1 * torch.randn(DV, generator=g)).numpy().astype(np.float32)
    return cw, A_log, dtb, gw


def rand_bf(gen, shape, scale=1.0):
    return (torch.randn(shape, generator=gen) * scale).bfloat16().float().numpy()


# ---- checks that fail with a short message (no array dumps)
def check_equal(name, a, b):
    a, b = np.asarray(a), np.asarray(b)
    if a.shape != b.shape:
        raise AssertionError(f"{name}: shape {a.shape} != {b.shape}")
    bad = a != b
    if a.dtype.kind == "f":
        bad &= ~(np.isnan(a) & np.isnan(b))
    n = int(bad.sum())
    if n:
        i = tuple(int(x) for x in np.argwhere(bad)[0])
        raise AssertionError(f"{name}: {n} of {a.size} elements differ; first at {i}: {a[i]!r} vs {b[i]!r}")


def check_ulp(name, got, ref, ulps=1.0, max_frac=None, rel_floor=1e-5):
    """|got - ref| <= ulps bf16 ulp of ref, plus rel_floor * max|ref| for results that are small by cancellation in a
    float32 dot product (and at most max_frac of the elements differ at all)"""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    bad = d > ulps * ulp_bf16(ref) + rel_floor * np.abs(ref).max() + 1e-30
    if bad.any():
        i = tuple(int(x) for x in np.argwhere(bad)[0])
        raise AssertionError(f"{name}: {int(bad.sum())} of {got.size} elements off by more than {ulps} bf16 ulp; first at {i}: "
                             f"{got[i]!r} vs {ref[i]!r}")
    if max_frac is not None and (d > 0).mean() > max_frac:
        raise AssertionError(f"{name}: {(d > 0).mean():.4f} of the elements differ (allowed {max_frac})")


def check_rel(name, got, ref, tol, measure=rel_max):
    e = measure(got, ref)
    if not e <= tol:
        raise AssertionError(f"{name}: relative error {e:.3e} > {tol:.1e}")
    return e


def check_tensors_equal(name, a, b):
    """bitwise equality of two torch tensors"""
    if a.shape != b.shape or a.dtype != b.dtype:
        raise AssertionError(f"{name}: {tuple(a.shape)} {a.dtype} vs {tuple(b.shape)} {b.dtype}")
    n = int((a != b).sum().item())
    if n:
        raise AssertionError(f"{name}: {n} of {a.numel()} elements differ")
