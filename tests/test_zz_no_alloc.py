"""The allocation-free decode / verify attention entry point (qt_gqa_attn_decode_static: partial results in a static device
array) against qt_gqa_attn_decode with a caller-owned workspace, both called through the C ABI: bit-identical outputs and pools,
on two calls in a row of which the second is smaller (the array keeps the first call's contents), and the size limit."""
import ctypes

import numpy as np
import pytest
import torch

from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu


def _case(lib, dev, seed, B, M, Lmax, lo, hi):
    rng = np.random.default_rng(seed)
    S = B + 2
    slots = rng.permutation(S)[:B].astype(np.int32)
    pos = rng.integers(lo, hi, B).astype(np.int32)
    Kp = to_dev(bf(rng.standard_normal((S + 1, 2, Lmax, 256))), dev, BF16)
    Vp = to_dev(bf(rng.standard_normal((S + 1, 2, Lmax, 256))), dev, BF16)
    q = to_dev(bf(rng.standard_normal((B * M, 8, 256))), dev, BF16)
    kn = to_dev(bf(rng.standard_normal((B * M, 2, 256))), dev, BF16)
    vn = to_dev(bf(rng.standard_normal((B * M, 2, 256))), dev, BF16)
    dslots, dpos = to_dev(slots, dev), to_dev(pos, dev)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    CH = 128
    # reference: the entry point with a workspace
    K1, V1 = Kp.clone(), Vp.clone()
    o1 = torch.zeros((B * M, 8, 256), dtype=BF16, device=dev)
    nws = lib.qt_gqa_attn_workspace_bytes(B, M, Lmax, CH)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    rc = lib.qt_gqa_attn_decode(p(q), p(kn), p(vn), p(K1), p(V1), p(dslots), p(dpos), p(o1), p(ws), nws, B, M, Lmax, S + 1, CH, stream)
    assert rc == 0, rc
    # the allocation-free one
    K2, V2 = Kp.clone(), Vp.clone()
    o2 = torch.zeros((B * M, 8, 256), dtype=BF16, device=dev)
    # a first call on scratch pools: the symbol lookup and the lazy load of the kernels' code object happen there, once
    K3, V3, o3 = Kp.clone(), Vp.clone(), torch.zeros_like(o2)
    rc = lib.qt_gqa_attn_decode_static(p(q), p(kn), p(vn), p(K3), p(V3), p(dslots), p(dpos), p(o3), B, M, Lmax, S + 1, CH, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)           # torch's caching allocator ...
    free_before = torch.cuda.mem_get_info(dev)[0]       # ... and the driver's own count of free device memory (sees a hipMalloc)
    rc = lib.qt_gqa_attn_decode_static(p(q), p(kn), p(vn), p(K2), p(V2), p(dslots), p(dpos), p(o2), B, M, Lmax, S + 1, CH, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before, "the driver's free-memory count moved across the call"
    check_tensors_equal(f"out (B={B}, M={M})", o2, o1)
    check_tensors_equal("K pool", K2, K1)
    check_tensors_equal("V pool", V2, V1)
    assert float(o1.float().abs().max()) > 0


def test_static_scratch_entry_point_matches_workspace_entry_point(dev):
    import qwen_tailor_amd as qt
    lib = qt._lib.lib()
    _case(lib, dev, 1, 16, 4, 4096 + 8, 1024, 4096)       # fills most of the partial slots
    _case(lib, dev, 2, 3, 1, 512, 0, 300)                 # smaller, right after: stale partials of the first call must not matter
    _case(lib, dev, 3, 128, 2, 256, 0, 250)               # the largest batch the static array takes
    _case(lib, dev, 4, 5, 7, 300, 0, 290)                 # more than four tokens per sequence: two passes over one array


def test_static_scratch_entry_point_rejects_larger_batches(dev):
    import qwen_tailor_amd as qt
    lib = qt._lib.lib()
    t = torch.zeros(16, dtype=torch.int32, device=dev)
    p = ctypes.c_void_p(t.data_ptr())
    rc = lib.qt_gqa_attn_decode_static(p, p, p, p, p, p, p, p, 129, 1, 64, 4, 128, ctypes.c_void_p(0))
    assert rc == -7
    assert qt._lib.ERRORS[-7].startswith("size beyond the maximum")
