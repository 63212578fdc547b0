"""The operators under HIP graph capture, the launch form bench.py times: each graph is replayed several times, with eager work
and synchronisations of the program's own between the replays, and every replay is compared bit for bit with the eager result
(operators that update pools in place start every replay from a restored pool)."""
import numpy as np
import pytest
import torch

from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    q._lib.lib()
    return q


def _replays(dev, run, outputs, restore=None, n=3):
    """eager reference, then a captured graph replayed n times; `outputs()` returns the tensors to compare"""
    if restore:
        restore()
    run()
    torch.cuda.synchronize()
    want = [t.clone() for t in outputs()]
    side = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        if restore:
            restore()
        run()                                         # once on the capture stream: per-stream scratch exists before the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=side):
            run()
    torch.cuda.synchronize()
    noise = torch.randn(1 << 20, device=dev)
    for i in range(n):
        if restore:
            restore()
        for t in outputs():
            if not restore:
                t.fill_(0)                            # a replay must write every output itself
        noise.mul_(1.0001)                            # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for k, (a, b) in enumerate(zip(outputs(), want)):
            check_tensors_equal(f"replay {i}, output {k}", a, b)


def test_decode_step_and_layer_half_under_graph(qt, dev):
    gen = torch.Generator().manual_seed(5)
    cw, A_log, dtb, gw = layer_params(31)
    B = 8
    ssm0 = to_dev((torch.randn((B + 1, 16, 128, 128), generator=gen) * 0.02).numpy(), dev)
    conv0 = to_dev(rand_bf(gen, ((B + 1) * 2, 3, CD)), dev, BF16)
    ssm, conv = ssm0.clone(), conv0.clone()
    x = to_dev(rand_bf(gen, (B, 1024)), dev, BF16)
    Wi = to_dev(rand_bf(gen, (PW, 1024), 0.03), dev, BF16)
    Wo = to_dev(rand_bf(gen, (1024, 2048), 0.02), dev, BF16)
    ln = to_dev(bf(1 + 0.1 * torch.randn(1024, generator=gen).numpy()), dev, BF16)
    slots = torch.randperm(B, generator=gen).to(torch.int32).to(dev)
    pos = torch.randint(0, 100, (B,), generator=gen).to(torch.int32).to(dev)
    dcw, dA, ddt, dgw = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev)
    out = torch.zeros((B, 1024), dtype=BF16, device=dev)

    def restore():
        ssm.copy_(ssm0)
        conv.copy_(conv0)

    def run():                                        # the GatedDeltaNet half of a layer at a decode step (batch.py:496-501)
        proj = qt.kernels.fused_gemv(Wi, qt.batch.rms_rows(x, ln))
        yn = qt.batch.deltanet_b_gnorm(proj, conv, dcw, dA, ddt, ssm, slots, pos, dgw)
        out.copy_(qt.kernels.fused_gemv(Wo, yn, res=x))
    _replays(dev, run, lambda: [out, ssm, conv], restore)


@pytest.mark.parametrize("T", [300, 4100])
def test_chunked_prefill_under_graph(qt, dev, T):
    """both launch forms of phase B; the one-launch form's flag area must be back to zero after every replay"""
    gen = torch.Generator().manual_seed(6 + T)
    cw, A_log, dtb, gw = layer_params(32)
    proj = to_dev(rand_bf(gen, (T, PW)), dev, BF16)
    cs = to_dev(rand_bf(gen, (1, 3, CD)), dev, BF16)
    S0 = to_dev((torch.randn((1, 16, 128, 128), generator=gen) * 0.02).numpy(), dev)
    dcw, dA, ddt, dgw = to_dev(cw, dev, BF16), to_dev(A_log, dev), to_dev(dtb, dev), to_dev(gw, dev)
    o = torch.zeros((T, 2048), dtype=BF16, device=dev)
    s1 = torch.zeros((1, 16, 128, 128), device=dev)
    c1 = torch.zeros((1, 3, CD), dtype=BF16, device=dev)

    def run():
        a, b, c = qt.prefill.gdn_core(proj, cs, S0, dcw, dA, ddt, dgw)
        o.copy_(a)
        c1.copy_(b)
        s1.copy_(c)
    _replays(dev, run, lambda: [o, s1, c1])
    flag_halves = qt._lib.lib().qt_gdn_chunk_snap_bytes(0) // 2
    for snap in qt.gdn_nax._SNAP.values():
        assert int(snap[:flag_halves].view(torch.int32).ne(0).sum().item()) == 0


@pytest.mark.parametrize("M", [1, 4, 6])
def test_decode_attention_under_graph(qt, dev, M):
    """attn_b and the two-launch layer form, pools restored before every replay (the new rows are appended in place)"""
    rng = np.random.default_rng(40 + M)
    B, Lmax = 6, 700
    slots = to_dev(rng.permutation(B).astype(np.int32), dev)
    pos = to_dev(rng.integers(0, Lmax - M, B).astype(np.int32), dev)
    K0 = to_dev(bf(rng.standard_normal((B + 1, 2, Lmax, 256))), dev, BF16)
    V0 = to_dev(bf(rng.standard_normal((B + 1, 2, Lmax, 256))), dev, BF16)
    Kp, Vp = K0.clone(), V0.clone()
    qkv = to_dev(bf(rng.standard_normal((B * M, 5120))), dev, BF16)
    qn, kn = to_dev(bf(1 + 0.1 * rng.standard_normal(256)), dev, BF16), to_dev(bf(1 + 0.1 * rng.standard_normal(256)), dev, BF16)
    o = torch.zeros((B * M, 2048), dtype=BF16, device=dev)
    o2 = torch.zeros((B * M, 2048), dtype=BF16, device=dev)
    qt.batch.attn_layer_b(qkv, qn, kn, Kp, Vp, slots, pos, M)          # builds the rotary table outside any capture

    def restore():
        Kp.copy_(K0)
        Vp.copy_(V0)

    def run_layer():
        o.copy_(qt.batch.attn_layer_b(qkv, qn, kn, Kp, Vp, slots, pos, M))

    def run_three():
        q, k, v = qt.attention.qkv_prep(qkv, qn, kn, pos, M)
        o2.copy_(qt.attention.out_gate(qt.batch.attn_b(q, k, v, Kp, Vp, slots, pos, M), qkv))
    _replays(dev, run_layer, lambda: [o, Kp, Vp], restore)
    _replays(dev, run_three, lambda: [o2, Kp, Vp], restore)
    check_tensors_equal("layer form == three calls", o, o2)


def test_prefill_attention_under_graph(qt, dev):
    rng = np.random.default_rng(50)
    S, L = 320, 1500                                  # rows continuing a prefix: the key-split form with its workspace
    q = to_dev(bf(rng.standard_normal((1, 8, S, 256))), dev, BF16)
    K = to_dev(bf(rng.standard_normal((1, 2, L, 256))), dev, BF16)
    V = to_dev(bf(rng.standard_normal((1, 2, L, 256))), dev, BF16)
    o = torch.zeros((1, 8, S, 256), dtype=BF16, device=dev)

    def run():
        o.copy_(qt.attention.scaled_dot_product_attention(q, K, V, scale=256 ** -0.5, mask="causal"))
    _replays(dev, run, lambda: [o])
