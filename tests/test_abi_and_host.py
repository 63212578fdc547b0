"""CPU-side checks: the C-ABI library loads and exports every symbol include/qwen_tailor_hip.h declares, the host layer
validates its arguments before anything reaches the GPU, and nothing in the product imports the oracle."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "qwen_tailor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import qwen_tailor_amd as qt
    lib = qt._lib.lib()
    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/qwen_tailor_hip.h but not exported"


def test_every_exported_entry_point_is_declared():
    import subprocess
    import qwen_tailor_amd as qt
    out = subprocess.run(["nm", "-D", "--defined-only", qt._build.SO], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r"\bT (qt_[a-z0-9_]+)", out)))
    assert exported == declared_symbols()


def test_host_rejects_bad_arguments_without_a_gpu():
    import qwen_tailor_amd as qt
    x = torch.zeros((2, 8224), dtype=torch.bfloat16)
    with pytest.raises(TypeError):                 # CPU tensors never reach the C ABI (no CPU fallback exists)
        qt.batch.deltanet_b(x, x, x, x, x, x, x, x)
    with pytest.raises(TypeError):
        qt.prefill.conv_prep(x, x, x)
    with pytest.raises(TypeError):
        qt.batch.attn_b(x, x, x, x, x, x, x)
    with pytest.raises(TypeError):
        qt.kernels.fused_gemv(x, x)
    with pytest.raises(TypeError):
        qt.batch.rms_rows(x, x[0])


def test_null_and_dimension_errors_from_the_c_abi():
    import qwen_tailor_amd as qt
    lib = qt._lib.lib()
    z = ctypes.c_void_p(0)
    assert lib.qt_gdn_decode_step(z, z, z, z, z, z, z, z, z, 1, 1, 0, z) == -3
    assert lib.qt_gqa_attn_workspace_bytes(16, 1, 32768, 1024) == (1024 + 16 * 2) * 4 * 258 * 4 + 8208   # partial results + segment table
    assert lib.qt_gqa_attn_workspace_bytes(1, 0, 16, 16) == -1
    assert lib.qt_normalize_qk(ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), ctypes.c_void_p(16), 1, 64, z) == -4
    p16 = ctypes.c_void_p(16)
    assert lib.qt_gdn_decode_step_gnorm(z, z, z, z, z, z, z, z, z, 1e-6, z, 1, 1, z) == -3
    assert lib.qt_blit(z, p16, 2, 8, 0, 0, 1, 0, 0, z) == -3
    assert lib.qt_blit(p16, p16, 3, 8, 0, 0, 1, 0, 0, z) == -4                       # element size 2 or 4 only
    assert lib.qt_blit(p16, p16, 2, -1, 0, 0, 1, 0, 0, z) == -1
    assert lib.qt_blit(p16, p16, 2, 0, 0, 0, 1, 0, 0, z) == 0                        # nothing to copy: no launch
    assert lib.qt_attn_qkv_prep(p16, p16, p16, p16, p16, p16, p16, 6, 4, 1e-6, z) == -1      # M must divide the rows
    assert lib.qt_attn_qkv_prep(p16, p16, p16, z, p16, p16, p16, 4, 4, 1e-6, z) == -3
    assert lib.qt_attn_qkv_prep_table(p16, p16, p16, p16, z, 0, p16, p16, p16, 6, 4, 1e-6, z) == -1
    assert lib.qt_attn_qkv_prep_table(p16, p16, p16, p16, p16, -1, p16, p16, p16, 4, 4, 1e-6, z) == -1
    assert lib.qt_attn_out_gate(p16, ctypes.c_void_p(8), p16, 1, z) == -2
    assert lib.qt_gdn_phase_a_conv(p16, p16, p16, p16, p16, p16, p16, z, z, z, p16, p16, p16, 64, z) == -3   # q without k, v
    assert lib.qt_gdn_phase_a_conv(p16, p16, p16, p16, p16, p16, z, z, z, p16, p16, p16, p16, 64, z) == -4   # conv_out aliases conv_state
    assert lib.qt_gqa_attn_decode(p16, p16, p16, p16, p16, p16, p16, p16, p16, 1 << 40, 2000, 1, 64, 1, 128, z) == -4   # B * 2 > 2048 segments
    assert lib.qt_rms_rows(p16, z, p16, 4, 1024, 1e-6, z) == -3
    assert lib.qt_rms_rows(p16, p16, p16, 4, 1020, 1e-6, z) == -1                    # K must be a multiple of 8
    assert lib.qt_rms_rows(p16, p16, p16, 0, 1024, 1e-6, z) == 0
    assert lib.qt_fused_gemv(p16, p16, z, p16, 4, 64, 1024, 1, z) == -3              # the add epilogue needs res
    assert lib.qt_fused_gemv(p16, p16, z, p16, 4, 64, 1000, 0, z) == -1              # K must be a multiple of 256
    assert lib.qt_fused_gemv(p16, p16, z, p16, 4, 63, 1024, 2, z) == -1              # swiglu pairs rows
    assert lib.qt_fused_gemv(p16, p16, z, p16, 4, 64, 1024, 3, z) == -4
    assert lib.qt_fused_gemv(p16, z, z, z, 0, 64, 1024, 1, z) == 0                   # no rows: nothing is dereferenced
    assert lib.qt_fused_gemv(ctypes.c_void_p(8), p16, z, p16, 4, 64, 1024, 0, z) == -2


def test_prefill_attention_split_plan_on_the_host():
    """The key split of the causal prefill attention is planned on the host (no GPU call computes anything here): which launches
    are split, how much workspace they use, and that the bound for a key count covers every launch below it."""
    import qwen_tailor_amd as qt
    lib = qt._lib.lib()
    need, bound = lib.qt_gqa_prefill_workspace_bytes_for, lib.qt_gqa_prefill_workspace_bytes
    z, p16 = ctypes.c_void_p(0), ctypes.c_void_p(16)
    assert need(-1, 8, 0) == -1 and need(8, 0, 0) == -1 and bound(-1) == -1
    assert need(4096, 4096, 0) == 0 and need(8192, 8192, 0) == 0          # a workgroup per CU or more: not split
    assert need(0, 64, 64) == 0 and need(5, 5, 0) == 0                    # nothing to split
    part = 4 * (16 * 256 * 2 + 2 * 16 * 4)                                # bytes of one part: O (half precision), m, l (float) of 16 rows x 4 heads
    for S, P0 in ((64, 8000), (16, 32000), (1024, 0), (1536, 1000), (300, 4001), (1, 4095), (2048, 0), (2048, 6000)):
        n = need(S, S + P0, P0)
        size = part * (2 if S >= 1472 else 1)                             # from about 1500 rows on the row blocks are 32 rows
        assert n > 0 and n % (2 * size) == 0, (S, P0, n)                  # whole parts, the same number for both KV heads
        assert n // size <= 256 + 1, (S, P0, n)                           # all parts resident at once (at most one per CU; 256 CUs assumed without a GPU)
        assert n <= bound(S + P0), (S, P0)
    # queries past the keys are refused before anything is launched
    assert lib.qt_gqa_prefill_causal(p16, p16, p16, p16, z, 0, 32, 40, 9, 32 * 256, 40 * 256, z) == -1
    assert lib.qt_gqa_prefill_causal(p16, p16, p16, p16, ctypes.c_void_p(8), 0, 32, 40, 8, 32 * 256, 40 * 256, z) == -2


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "qwen-tailor_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"(from|import)\s+oracle|oracle[/.]|libgdn_oracle", text), f"{f} reaches into oracle/"


def test_pools_shapes_and_byte_accounting():
    """Pools / SpecPools layouts and slot_bytes (qwen35/batch.py:405-426, qwen35/batch_spec.py:242-270) on the CPU device."""
    import qwen_tailor_amd as qt
    cfg = qt.model.Cfg()
    assert cfg.conv_dim == 6144 and sum(cfg.is_linear(i) for i in range(cfg.layers)) == 18
    P = qt.batch.Pools(cfg, 3, 64, device="cpu")
    assert len(P.ssm) == 18 and len(P.K) == 6
    assert tuple(P.ssm[0].shape) == (4, 16, 128, 128) and tuple(P.conv[0].shape) == (8, 3, 6144)
    assert tuple(P.K[0].shape) == (4, 2, 64, 256)
    assert P.nbytes() == 4 * qt.batch.Pools.slot_bytes(cfg, 64)
    assert qt.batch.Pools.slot_bytes(cfg, 64, double_conv=False) == 18 * (16 * 128 * 128 * 4 + 3 * 6144 * 2) + 6 * 2 * 2 * 64 * 256 * 2
    st = {"conv": [torch.randn(1, 3, 6144).bfloat16() for _ in range(18)], "ssm": [torch.randn(1, 16, 128, 128) for _ in range(18)],
          "kv": [(torch.randn(1, 2, 64, 256).bfloat16(), torch.randn(1, 2, 64, 256).bfloat16()) for _ in range(6)]}
    # the load -> read round trip (tests/batch.py:102-112) runs the copy kernel: tests/test_state_blit_gpu.py; without a GPU
    # the operator must fail loudly rather than copy on the host
    with pytest.raises(TypeError):
        P.load(2, st, 37)
    with pytest.raises(AssertionError):
        P.load(3, st, 1)                                    # the trash slot cannot be loaded (batch.py:434)
    SP = qt.batch_spec.SpecPools(cfg, 2, 3, 4, 64, device="cpu")
    assert tuple(SP.ssm[0].shape) == (3, 4, 16, 128, 128) and tuple(SP.conv[0].shape) == (6, 4, 3, 6144)
    assert qt.batch_spec.SpecPools.entry_bytes(cfg, 4) == 18 * 4 * (16 * 128 * 128 * 4 + 2 * 3 * 6144 * 2)
