"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py): the CPU oracle must reproduce them bit
for bit (CPU test), and the HIP kernels must match them to the path's tolerances (GPU tests)."""
import os

import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from tests.util import *  # noqa: F401,F403

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def unbits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def decode_inputs():
    z = np.load(os.path.join(G, "decode_step.npz"))
    gen = torch.Generator().manual_seed(int(z["seed"]))
    cw, A_log, dtb, gw = layer_params(int(z["seed"]))
    proj = rand_bf(gen, (3, PW))
    conv = rand_bf(gen, (8, 3, CD))
    ssm = (torch.randn((4, 16, 128, 128), generator=gen) * 0.02).numpy()
    assert np.array_equal(proj, unbits(z["proj"])) and np.array_equal(conv, unbits(z["conv"]))
    return z, cw, A_log, dtb, gw, proj, conv, ssm


def prefill_inputs():
    z = np.load(os.path.join(G, "prefill_gdn.npz"))
    gen = torch.Generator().manual_seed(int(z["seed"]))
    cw, A_log, dtb, gw = layer_params(int(z["seed"]))
    T = int(z["T"])
    proj = rand_bf(gen, (T, PW))
    cs = rand_bf(gen, (3, CD))
    S0 = (torch.randn((16, 128, 128), generator=gen) * 0.02).numpy()
    return z, cw, A_log, dtb, gw, proj, cs, S0


def test_oracle_reproduces_fixtures():
    z, cw, A_log, dtb, gw, proj, conv, ssm = decode_inputs()
    y = O.deltanet_b(proj, conv, cw, A_log, dtb, ssm, z["slots"], z["pos"])
    check_equal("decode y", y, unbits(z["y"]))
    check_equal("decode conv pool", conv, unbits(z["conv_out"]))
    check_equal("decode state", ssm[:3][:, z["heads"]], z["ssm_out_heads"])
    check_equal("decode gated norm", O.gated_norm(y, proj, gw), unbits(z["out"]))
    z, cw, A_log, dtb, gw, proj, cs, S0 = prefill_inputs()
    out, y, tail, S1 = O.prefill_gdn(proj, cs, cw, A_log, dtb, S0, gw)
    check_equal("prefill y", y, unbits(z["y"]))
    check_equal("prefill out", out, unbits(z["out"]))
    check_equal("prefill conv tail", tail, unbits(z["tail"]))
    check_equal("prefill state", S1[z["heads"]], z["S1_heads"])
    q, k, v = O.conv_prep(proj, cs, cw)
    check_equal("prefill q", q[:, z["heads"]], unbits(z["q"]))
    check_equal("prefill k", k[:, z["heads"]], unbits(z["k"]))
    z = np.load(os.path.join(G, "attention.npz"))
    o = O.attn_b(unbits(z["q"]), unbits(z["kn"]), unbits(z["vn"]), unbits(z["Kp"]), unbits(z["Vp"]), z["slots"], z["pos"], int(z["M"]))
    check_equal("attn_b", o, unbits(z["o"]))
    check_equal("sdpa_causal", O.sdpa_causal(unbits(z["qc"]), unbits(z["Kc"]), unbits(z["Vc"])), unbits(z["oc"]))
    z = np.load(os.path.join(G, "attn_glue.npz"))
    q, k, v = O.attn_qkv_prep(unbits(z["qkv"]), unbits(z["q_norm"]), unbits(z["k_norm"]), z["pos"], int(z["M"]))
    check_equal("glue q", q, unbits(z["q"]))
    check_equal("glue k", k, unbits(z["k"]))
    check_equal("glue v", v, unbits(z["v"]))
    check_equal("glue gate", O.attn_out_gate(unbits(z["o"]), unbits(z["qkv"])), unbits(z["gated"]))
    z = np.load(os.path.join(G, "projections.npz"))
    x, nw, W1, Wg = (unbits(z[n]) for n in ("x", "nw", "W1", "Wg"))
    check_equal("rms_rows", O.rms_rows(x, nw), unbits(z["xn"]))
    check_equal("gemv rms", O.fused_gemv(W1, x, nw=nw), unbits(z["y_rms"]))
    check_equal("gemv add", O.fused_gemv(W1, x, res=unbits(z["res"])), unbits(z["y_add"]))
    check_equal("gemv swiglu", O.fused_gemv(Wg, x, swiglu=True), unbits(z["y_swiglu"]))


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    q._lib.lib()
    return q


@pytest.mark.gpu
def test_decode_step_matches_fixture(qt, dev):
    z, cw, A_log, dtb, gw, proj, conv, ssm = decode_inputs()
    dconv, dssm, dproj = to_dev(conv, dev, BF16), to_dev(ssm, dev), to_dev(proj, dev, BF16)
    y = qt.batch.deltanet_b(dproj, dconv, to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), dssm, to_dev(z["slots"], dev),
                            to_dev(z["pos"], dev))
    check_equal("conv pool", to_np(dconv), unbits(z["conv_out"]))
    check_rel("state", to_np(dssm)[:3][:, z["heads"]], z["ssm_out_heads"], 1e-4, rel_max)
    check_ulp("y", to_np(y), unbits(z["y"]))
    check_ulp("gated norm of the oracle's y", to_np(qt.batch.gnorm_rows(to_dev(unbits(z["y"]), dev, BF16), dproj, to_dev(gw, dev))),
              unbits(z["out"]), ulps=0)


@pytest.mark.gpu
def test_prefill_matches_fixture(qt, dev):
    z, cw, A_log, dtb, gw, proj, cs, S0 = prefill_inputs()
    T = int(z["T"])
    for impl in ("nax", "ref"):                                                # chunked MFMA kernels and the sequential kernel
        qt.prefill.GDN_IMPL = impl
        out, new_conv, new_ssm = qt.prefill.gdn_core(to_dev(proj, dev, BF16), to_dev(cs[None], dev, BF16), to_dev(S0[None], dev),
                                                     to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev))
        check_equal(f"{impl}: new conv state", to_np(new_conv)[0], unbits(z["tail"]))
        check_rel(f"{impl}: state", to_np(new_ssm)[0][z["heads"]], z["S1_heads"], 2e-3, rel_l2)
        check_rel(f"{impl}: gated output", to_np(out), unbits(z["out"]), 2e-3, rel_l2)
    qt.prefill.GDN_IMPL = "nax"
    q, k, v = qt.prefill.conv_prep(to_dev(proj, dev, BF16), to_dev(cs, dev, BF16), to_dev(cw, dev, BF16))
    check_equal("q", to_np(q)[:, z["heads"]], unbits(z["q"]))
    check_equal("k", to_np(k)[:, z["heads"]], unbits(z["k"]))
    check_equal("v", to_np(v)[:, z["heads"]], unbits(z["v"]))


@pytest.mark.gpu
def test_attention_matches_fixture(qt, dev):
    z = np.load(os.path.join(G, "attention.npz"))
    d = lambda name: to_dev(unbits(z[name]), dev, BF16)
    o = qt.batch.attn_b(d("q"), d("kn"), d("vn"), d("Kp"), d("Vp"), to_dev(z["slots"], dev), to_dev(z["pos"], dev), int(z["M"]))
    check_rel("attn_b", to_np(o), unbits(z["o"]), 1e-2, rel_l2)
    oc = qt.attention.scaled_dot_product_attention(d("qc")[None], d("Kc")[None], d("Vc")[None], scale=256 ** -0.5, mask="causal")
    check_rel("causal prefill", to_np(oc)[0], unbits(z["oc"]), 1e-2, rel_l2)


@pytest.mark.gpu
def test_attention_glue_matches_fixture(qt, dev):
    z = np.load(os.path.join(G, "attn_glue.npz"))
    d = lambda name: to_dev(unbits(z[name]), dev, BF16)
    q, k, v = qt.attention.qkv_prep(d("qkv"), d("q_norm"), d("k_norm"), to_dev(z["pos"], dev), int(z["M"]))
    check_equal("q", to_np(q), unbits(z["q"]))
    check_equal("k", to_np(k), unbits(z["k"]))
    check_equal("v", to_np(v), unbits(z["v"]))
    check_equal("gated output", to_np(qt.attention.out_gate(d("o"), d("qkv"))), unbits(z["gated"]))


@pytest.mark.gpu
def test_projections_match_fixture(qt, dev):
    """rms_rows bit for bit; the products within one bf16 rounding step (two after the second rounding of add / swiglu) plus the
    float32 accumulation error of sums that nearly cancel"""
    z = np.load(os.path.join(G, "projections.npz"))
    d = lambda name: to_dev(unbits(z[name]), dev, BF16)
    check_equal("rms_rows", to_np(qt.batch.rms_rows(d("x"), d("nw"))), unbits(z["xn"]))

    def close(name, got, want, ulps):
        got, want = to_np(got).astype(np.float64), unbits(z[want]).astype(np.float64)
        bad = np.abs(got - want) > ulps * ulp_bf16(np.maximum(np.abs(got), np.abs(want))) + 2e-5 * np.abs(want).max()
        assert not bad.any(), f"{name}: {int(bad.sum())} outputs off"
    close("rms + product", qt.kernels.fused_gemv(d("W1"), d("x"), nw=d("nw")), "y_rms", 1)
    close("add", qt.kernels.fused_gemv(d("W1"), d("x"), res=d("res")), "y_add", 2)
    close("swiglu", qt.kernels.fused_gemv(d("Wg"), d("x"), swiglu=True), "y_swiglu", 2)
