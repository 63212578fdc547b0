"""Headline benchmark: batched GatedDeltaNet decode step at B=64 (HBM roofline), one GPU.

A "step" is one launch of the fused decode kernel for one layer's pools: 64 rows, each reading and writing its 16 x 64 KiB
float32 state in place.  The launches rotate over 18 independent layer pools (1.15 GiB of state, as the real model does) so
the state cannot stay in the 256 MB last-level cache; the single-pool (cache-resident) rate is reported separately.

Prints ONE JSON line (see README of the build contract): metric/value/unit, roofline, cpu_baseline, extras.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HV, DK, DV, CD, PW = 16, 128, 128, 6144, 8224
N_LAYERS = 18
HBM_PEAK_GBS = 8000.0
# HBM bytes of one B = 64 decode launch measured with rocprofv3 --pmc (FETCH_SIZE 34 564.9 KiB x 1.9993 + WRITE_SIZE 68 145.9 KiB,
# scale factors from a 64 MiB copy; profiles/gdn_decode_wide_kernel_B64.md).  Reported as `roofline.traffic` for that batch only.
DECODE_TRAFFIC_B64 = int((34564.9 * 1.9993 + 68145.9) * 1024)
DECODE_TRAFFIC_SOURCE = ("profiles/gdn_decode_wide_kernel_B64.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of gdn_decode_wide_kernel<4> at "
                         "B=64 (a recorded measurement of that kernel, not of this run)")
# same for the three kernels of the T = 2048 prefill (profiles/gdn_prefill_T2048.md)
PREFILL_TRAFFIC_T2048 = int(((16691.8 + 13314.7 + 23734.0) * 1.9993 + 37172.2 + 25600 + 8192) * 1024)
PREFILL_TRAFFIC_SOURCE = ("profiles/gdn_prefill_T2048.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of gdn_phase_a_kernel, gdn_chain_kernel and "
                          "gdn_output_kernel at T=2048 (a recorded measurement of those kernels, not of this run)")


def decode_bytes(B):
    """algorithmic HBM bytes of one decode step of one layer: state R+W, projection row, conv window R+W, y, conv weights"""
    return B * (2 * HV * DV * DK * 4 + PW * 2 + 2 * 3 * CD * 2 + 2048 * 2) + CD * 4 * 2


def build_decode_state(torch, dev, B, n_layers, seed=1001):
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    st = {
        "ssm": [(torch.randn((B + 1, HV, DV, DK), generator=g) * 0.02).to(dev) for _ in range(n_layers)],
        "conv": [torch.randn(((B + 1) * 2, 3, CD), generator=g).to(bf).to(dev) for _ in range(n_layers)],
        "cw": [(torch.randn((CD, 4), generator=g) * 0.5).to(bf).to(dev) for _ in range(n_layers)],
        "A_log": [(torch.rand(HV, generator=g) * 2.7).to(dev) for _ in range(n_layers)],
        "dtb": [(torch.randn(HV, generator=g) * 0.1).to(bf).float().to(dev) for _ in range(n_layers)],
        # hidden [B,1024] bf16 -> in_proj is a dense projection outside the path: the 8224-wide rows are drawn directly
        "proj": [torch.randn((B, PW), generator=g).to(bf).to(dev) for _ in range(4)],
        "slots": torch.randperm(B, generator=g).to(torch.int32).to(dev),
        "pos": [torch.full((B,), 300 + p, dtype=torch.int32).to(dev) for p in (0, 1)],
    }
    return st


def time_decode(torch, qt, st, B, n_layers, steps, warmup, use_graph=True, min_total_s=0.05, max_regions=400):
    """`warmup` untimed launches, then timed regions of exactly `steps` launches each, every region bracketed by a device
    synchronisation and by events on the launching stream.  One region of a few launches is shorter than the noise of its own
    bracket, so regions are repeated until they fill `min_total_s` and the MEDIAN region is reported, on each clock.  Returns
    (median wall seconds, median device seconds, regions)."""
    def model_step(par):
        for l in range(n_layers):
            qt.batch.deltanet_b(st["proj"][(l + par) & 3], st["conv"][l], st["cw"][l], st["A_log"][l], st["dtb"][l], st["ssm"][l],
                                st["slots"], st["pos"][par])

    def one(i):
        l = i % n_layers
        par = (i // n_layers) & 1
        qt.batch.deltanet_b(st["proj"][(l + par) & 3], st["conv"][l], st["cw"][l], st["A_log"][l], st["dtb"][l], st["ssm"][l],
                            st["slots"], st["pos"][par])

    graphs = None
    if use_graph:
        model_step(0)
        torch.cuda.synchronize()
        graphs = []
        s = torch.cuda.Stream()
        for par in (0, 1):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(s):
                with torch.cuda.graph(g, stream=s):
                    model_step(par)
            graphs.append(g)
        torch.cuda.synchronize()
        for _ in range(10):                              # set-up, not warm-up: a graph's first replays upload and settle it
            graphs[0].replay()
            graphs[1].replay()
        torch.cuda.synchronize()

    def run(n, start=0):
        i = start
        while n > 0:
            if graphs is not None and i % n_layers == 0 and n >= n_layers:
                graphs[(i // n_layers) & 1].replay()
                i += n_layers
                n -= n_layers
            else:
                one(i)
                i += 1
                n -= 1
        return i

    def align(i):
        return ((i + n_layers - 1) // n_layers) * n_layers if graphs is not None else i

    i = align(run(warmup))
    walls, devs, total = [], [], 0.0
    # regions alternate between the two clocks: an event record is a packet of its own on the stream, and inside a wall-clock
    # region of a few launches the two of them would be timed as if they were part of the work
    while min(len(walls), len(devs)) < 3 or (total < min_total_s and len(walls) + len(devs) < max_regions):
        torch.cuda.synchronize()
        if len(walls) <= len(devs):
            t0 = time.perf_counter()
            i = run(steps, i)
            torch.cuda.synchronize()
            walls.append(time.perf_counter() - t0)
            total += walls[-1]
        else:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            i = run(steps, i)
            e1.record()
            torch.cuda.synchronize()
            devs.append(e0.elapsed_time(e1) * 1e-3)
            total += devs[-1]
        i = align(i)
    dev_s = sorted(devs)[len(devs) // 2]
    wall = sorted(walls)[len(walls) // 2]
    return wall, dev_s, len(walls) + len(devs)


def time_graph(torch, fn, reps=200, inner=10):
    """average device time (s) of fn(), measured with events around replays of a HIP graph holding `inner` calls"""
    fn()
    torch.cuda.synchronize()
    st = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        fn()                                          # once on the capture stream: per-stream scratch buffers exist before the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=st):
            for _ in range(inner):
                fn()
    torch.cuda.synchronize()
    n = max(1, reps // inner)
    for _ in range(max(3, n // 2)):                   # warm-up replays: clocks and caches settle before the timed region
        g.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(n):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / (n * inner)


MFMA_PEAK_TFLOPS = 2500.0
GDN_FLOP_PER_TOKEN = 2621440.0        # 16 heads x (4 C^2 dk + 4 C^2 dv + 6 C dk dv) / C at C = 64, dk = dv = 128


LLC_BYTES = 256 << 20                 # last-level cache: an input set that is to come from HBM rotates over more bytes than this


def bench_prefill(torch, qt, dev, T, seed=1002):
    """benchmark config 2: conv + chunked GDN (chunk 64) + gated RMSNorm over T tokens from a nonzero state.  The calls rotate
    over enough independent input sets (projection rows, conv window, initial state) to exceed the last-level cache, so every
    call reads its rows from HBM; the records between the kernels are the library's scratch and stay where the hardware keeps
    them, as they do between the layers of a model."""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    set_bytes = T * PW * 2
    n_sets = max(8, -(-(LLC_BYTES + LLC_BYTES // 4) // set_bytes))
    base = torch.randn((T, PW), generator=g).to(bf)
    sets = []
    for i in range(n_sets):
        proj = torch.roll(base, shifts=i * 37, dims=0).to(dev)                 # same distribution, different rows at every address
        cs = torch.randn((1, 3, CD), generator=g).to(bf).to(dev)
        S0 = (torch.randn((1, HV, DV, DK), generator=g) * 0.02).to(dev)
        sets.append((proj, cs, S0))
    cw = (torch.randn((CD, 4), generator=g) * 0.5).to(bf).to(dev)
    A = (torch.rand(HV, generator=g) * 2.7).to(dev)
    dtb = (torch.randn(HV, generator=g) * 0.1).to(dev)
    gw = torch.ones(DV, device=dev)
    ops, U, gC = qt.gdn_nax._phase_a(sets[0][0], sets[0][1][0], cw, A, dtb, want_qkv=False)[3:]
    it = [0]

    def nxt():
        it[0] += 1
        return sets[it[0] % n_sets]

    def whole():
        proj, cs, S0 = nxt()
        qt.prefill.gdn_core(proj, cs, S0, cw, A, dtb, gw)

    def only_a():
        proj, cs, _ = nxt()
        qt.gdn_nax._phase_a(proj, cs[0], cw, A, dtb, want_qkv=False)

    def only_b():                                    # (one set of records, as phase A leaves them behind: they are the library's scratch)
        proj, _, S0 = nxt()
        qt.gdn_nax.phase_b_norm(proj, ops, U, gC, S0, gw)
    t_all = time_graph(torch, whole, reps=n_sets * 8, inner=n_sets)
    t_a = time_graph(torch, only_a, reps=n_sets * 8, inner=n_sets)
    t_b = time_graph(torch, only_b, reps=n_sets * 8, inner=n_sets)
    flop = GDN_FLOP_PER_TOKEN * T
    hbm = T * PW * 2 + T * 2048 * 2 + 2 * HV * DV * DK * 4          # compulsory: projection rows in, gated output out, state in + out
    return {"T": T, "input_sets": n_sets, "inputs": "rotated past the last-level cache", "tok_per_s": T / t_all, "us": t_all * 1e6,
            "conv_phase_a_us": t_a * 1e6, "chain_output_norm_us": t_b * 1e6, "mfma_tflops": flop / t_all / 1e12,
            "mfma_frac": flop / t_all / 1e12 / MFMA_PEAK_TFLOPS, "compulsory_hbm_GBps": hbm / t_all / 1e9}


def bench_verify_gdn(torch, qt, dev, B=16, M=4, seed=1004):
    """benchmark config 4, GDN half: B sequences x M draft tokens, a state snapshot after every token"""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    pools = [((torch.randn((B + 1, M, HV, DV, DK), generator=g) * 0.02).to(dev), torch.randn(((B + 1) * 2, M, 3, CD), generator=g).to(bf).to(dev))
             for _ in range(N_LAYERS)]
    proj = torch.randn((B * M, PW), generator=g).to(bf).to(dev)
    cw = (torch.randn((CD, 4), generator=g) * 0.5).to(bf).to(dev)
    A = (torch.rand(HV, generator=g) * 2.7).to(dev)
    dtb = (torch.randn(HV, generator=g) * 0.1).to(dev)
    ss = torch.randperm(B, generator=g).to(torch.int32).to(dev)
    sels = torch.randint(0, M, (B,), generator=g).to(torch.int32).to(dev)
    pars = torch.zeros(B, dtype=torch.int32, device=dev)
    it = [0]

    def step():
        ssm, conv = pools[it[0] % N_LAYERS]
        it[0] += 1
        qt.batch_spec.deltanet_bm(proj, conv, cw, A, dtb, ssm, ss, sels, pars, M)
    t = time_graph(torch, step, reps=N_LAYERS * 20, inner=N_LAYERS)
    nbytes = B * ((1 + M) * HV * DV * DK * 4 + M * PW * 2 + 3 * CD * 2 + M * 3 * CD * 2 + M * 2048 * 2)
    return {"B": B, "M": M, "us": t * 1e6, "bytes": nbytes, "GBps": nbytes / t / 1e9, "hbm_frac": nbytes / t / 1e9 / HBM_PEAK_GBS}


def bench_attn(torch, qt, dev, B, M, lo, hi, seed):
    """benchmark configs 3 / 4 (attention half): ragged KV lengths uniform in [lo, hi], M query rows per sequence"""
    import numpy as np
    rng = np.random.default_rng(seed)
    Lmax = hi + 8
    pos = torch.from_numpy(rng.integers(lo, hi, B).astype(np.int32)).to(dev)
    slots = torch.from_numpy(rng.permutation(B).astype(np.int32)).to(dev)
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    nbytes = int(pos.sum().item()) * 2 * 2 * 256 * 2                  # K and V rows of both KV heads, read once
    # a step's K / V must come from HBM, not from the 256 MB last-level cache: rotate over enough pools (layers) to exceed it
    n_pools = max(2, min(16, -(-1100000000 // nbytes)))
    Kp0 = torch.randn((B + 1, 2, Lmax, 256), generator=g).to(bf).to(dev)
    Vp0 = torch.randn((B + 1, 2, Lmax, 256), generator=g).to(bf).to(dev)
    pools = [(Kp0, Vp0)] + [(Kp0.clone(), Vp0.clone()) for _ in range(n_pools - 1)]
    q = torch.randn((B * M, 8, 256), generator=g).to(bf).to(dev)
    kn = torch.randn((B * M, 2, 256), generator=g).to(bf).to(dev)
    vn = torch.randn((B * M, 2, 256), generator=g).to(bf).to(dev)
    it = [0]

    def step():
        Kp, Vp = pools[it[0] % n_pools]
        it[0] += 1
        qt.batch.attn_b(q, kn, vn, Kp, Vp, slots, pos, M)
    t = time_graph(torch, step, reps=n_pools * 12, inner=n_pools)
    return {"B": B, "M": M, "pools": n_pools, "sum_L": int(pos.sum().item()), "us": t * 1e6, "bytes": nbytes, "GBps": nbytes / t / 1e9,
            "hbm_frac": nbytes / t / 1e9 / HBM_PEAK_GBS}


def bench_attn_layer(torch, qt, dev, B, M, lo, hi, seed):
    """the attention half of a full-attention layer at a decode / verify step, between its qkv and o projections
    (qwen35/batch.py:505-513): as attention.qkv_prep + batch.attn_b + attention.out_gate (four launches) and as
    batch.attn_layer_b (two); pools rotated as in bench_attn"""
    import numpy as np
    rng = np.random.default_rng(seed)
    Lmax = hi + 8
    pos = torch.from_numpy(rng.integers(lo, hi, B).astype(np.int32)).to(dev)
    slots = torch.from_numpy(rng.permutation(B).astype(np.int32)).to(dev)
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    nbytes = int(pos.sum().item()) * 2 * 2 * 256 * 2
    n_pools = max(2, min(16, -(-1100000000 // nbytes)))
    Kp0 = torch.randn((B + 1, 2, Lmax, 256), generator=g).to(bf).to(dev)
    Vp0 = torch.randn((B + 1, 2, Lmax, 256), generator=g).to(bf).to(dev)
    pools = [(Kp0, Vp0)] + [(Kp0.clone(), Vp0.clone()) for _ in range(n_pools - 1)]
    qkv = torch.randn((B * M, 5120), generator=g).to(bf).to(dev)
    qn, kn = torch.ones(256, dtype=bf, device=dev), torch.ones(256, dtype=bf, device=dev)
    it = [0]

    def four():
        Kp, Vp = pools[it[0] % n_pools]
        it[0] += 1
        q, k, v = qt.attention.qkv_prep(qkv, qn, kn, pos, M)
        qt.attention.out_gate(qt.batch.attn_b(q, k, v, Kp, Vp, slots, pos, M), qkv)

    def two():
        Kp, Vp = pools[it[0] % n_pools]
        it[0] += 1
        qt.batch.attn_layer_b(qkv, qn, kn, Kp, Vp, slots, pos, M)
    t4 = time_graph(torch, four, reps=n_pools * 12, inner=n_pools)
    t2 = time_graph(torch, two, reps=n_pools * 12, inner=n_pools)
    return {"B": B, "M": M, "pools": n_pools, "sum_L": int(pos.sum().item()), "four_launches_us": t4 * 1e6, "two_launches_us": t2 * 1e6,
            "bytes": nbytes, "two_launches_GBps": nbytes / t2 / 1e9, "two_launches_hbm_frac": nbytes / t2 / 1e9 / HBM_PEAK_GBS}


def bench_attn_prefill(torch, qt, dev, S=2048, seed=7):
    """causal prefill attention over S rows; the calls rotate over enough (q, K, V) sets to exceed the last-level cache"""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    set_bytes = (8 + 2 + 2) * S * 256 * 2
    n_sets = max(8, -(-(LLC_BYTES + LLC_BYTES // 4) // set_bytes))
    q0 = torch.randn((1, 8, S, 256), generator=g).to(bf)
    K0 = torch.randn((1, 2, S, 256), generator=g).to(bf)
    V0 = torch.randn((1, 2, S, 256), generator=g).to(bf)
    sets = [(torch.roll(q0, i * 5, 2).to(dev), torch.roll(K0, i * 3, 2).to(dev), torch.roll(V0, i * 7, 2).to(dev)) for i in range(n_sets)]
    it = [0]

    def step():
        q, K, V = sets[it[0] % n_sets]
        it[0] += 1
        qt.attention.scaled_dot_product_attention(q, K, V, scale=256 ** -0.5, mask="causal")
    t = time_graph(torch, step, reps=n_sets * 5, inner=n_sets)
    flop = 4.0 * S * S * 256 * 8 / 2
    return {"S": S, "input_sets": n_sets, "inputs": "rotated past the last-level cache", "us": t * 1e6, "tflops": flop / t / 1e12,
            "mfma_frac": flop / t / 1e12 / MFMA_PEAK_TFLOPS}


def bench_state_admission(torch, qt, dev, pos=2048, Lmax=4096, slots=8):
    """Admission of one prefilled sequence into its slot (Pools.load, qwen35/batch.py:431-447): 18 layers of recurrent state
    (1 MiB + 36 KiB each) and 6 layers of K / V rows (pos x 2 heads x 512 B each, twice), 60 strided copies."""
    cfg = qt.model.Cfg()
    P = qt.batch.Pools(cfg, slots, Lmax, device=dev)
    nl, na = len(P.conv), len(P.K)
    bf = torch.bfloat16
    state = {"conv": [torch.zeros((1, 3, CD), dtype=bf, device=dev) for _ in range(nl)],
             "ssm": [torch.zeros((1, HV, DV, DK), device=dev) for _ in range(nl)],
             "kv": [(torch.zeros((1, cfg.n_kv, pos, cfg.head_dim), dtype=bf, device=dev),
                     torch.zeros((1, cfg.n_kv, pos, cfg.head_dim), dtype=bf, device=dev)) for _ in range(na)]}
    it = [0]

    def step():
        P.load(it[0] % slots, state, pos)
        it[0] += 1
    t = time_graph(torch, step, reps=slots * 6, inner=slots)
    nbytes = 2 * (nl * (HV * DV * DK * 4 + 3 * CD * 2) + na * 2 * cfg.n_kv * pos * cfg.head_dim * 2)      # read + written
    return {"pos": pos, "copies": 2 * nl + 2 * na, "us": t * 1e6, "bytes": nbytes, "GBps": nbytes / t / 1e9,
            "hbm_frac": nbytes / t / 1e9 / HBM_PEAK_GBS}


def bench_attn_glue(torch, qt, dev, R=2048, seed=5):
    """q / k RMSNorm + partial RoPE + split (qkv_prep) and the output gate over R rows (R = 2048: one prefill's rows)"""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    qkv = torch.randn((R, 5120), generator=g).to(bf).to(dev)
    qn, kn = torch.ones(256, dtype=bf, device=dev), torch.ones(256, dtype=bf, device=dev)
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    o = torch.randn((R, 8, 256), generator=g).to(bf).to(dev)
    t1 = time_graph(torch, lambda: qt.attention.qkv_prep(qkv, qn, kn, pos, M=R), reps=60, inner=3)
    t1t = time_graph(torch, lambda: qt.attention.qkv_prep(qkv, qn, kn, pos, M=R, max_pos=R), reps=60, inner=3)   # rotary pairs from the table
    t2 = time_graph(torch, lambda: qt.attention.out_gate(o, qkv), reps=60, inner=3)
    b1, b2 = R * (3072 + 3072) * 2, R * (2048 * 3) * 2          # q, k, v columns in + out; o, gate in + out
    return {"rows": R, "qkv_prep_us": t1 * 1e6, "qkv_prep_GBps": b1 / t1 / 1e9, "qkv_prep_table_us": t1t * 1e6,
            "out_gate_us": t2 * 1e6, "out_gate_GBps": b2 / t2 / 1e9}


def bench_projections(torch, qt, dev, B=64, seed=9):
    """The projections either side of the GDN core at a decode step of B rows (hidden 1024): rms_rows + in_proj [8224 x 1024],
    and out_proj [1024 x 2048] with the residual (qwen35/batch.py:496-501); eight copies of each weight rotate so that no copy
    stays in the last-level cache between uses less than the layer count apart."""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    Wi = [(torch.randn((PW, 1024), generator=g) / 32).to(bf).to(dev) for _ in range(8)]
    Wo = [(torch.randn((1024, 2048), generator=g) / 45).to(bf).to(dev) for _ in range(8)]
    x = torch.randn((B, 1024), generator=g).to(bf).to(dev)
    ln = torch.ones(1024, dtype=bf, device=dev)
    yn = torch.randn((B, 2048), generator=g).to(bf).to(dev)
    it = [0]

    def in_proj():
        qt.kernels.fused_gemv(Wi[it[0] % 8], qt.batch.rms_rows(x, ln))
        it[0] += 1

    def out_proj():
        qt.kernels.fused_gemv(Wo[it[0] % 8], yn, res=x)
        it[0] += 1
    t0 = time_graph(torch, lambda: qt.batch.rms_rows(x, ln), reps=40, inner=8)
    t1 = time_graph(torch, in_proj, reps=40, inner=8)
    t2 = time_graph(torch, out_proj, reps=40, inner=8)
    b1 = PW * 1024 * 2 + B * (1024 * 2 * 3 + PW * 2)
    b2 = 1024 * 2048 * 2 + B * (2048 * 2 + 1024 * 2 * 2)
    return {"B": B, "rms_rows_us": t0 * 1e6, "rms_in_proj_us": t1 * 1e6, "rms_in_proj_GBps": b1 / t1 / 1e9,
            "out_proj_add_us": t2 * 1e6, "out_proj_add_GBps": b2 / t2 / 1e9}


def bench_prefix_cache(torch, qt, dev, pos=2048, max_len=4096):
    """A prefix-cache checkpoint of a prefilled sequence (qwen35/prefix_cache.py:157-188: 12 K / V segments of `pos` rows + 18
    recurrent states, one launch) and its restore into fresh max_len buffers (prefix_cache.py:139-154)."""
    import numpy as np
    cfg = qt.model.Cfg()
    nl = sum(cfg.is_linear(i) for i in range(cfg.layers))
    na = cfg.layers - nl
    bf = torch.bfloat16
    st = {"kv": [(torch.zeros((1, cfg.n_kv, max_len, cfg.head_dim), dtype=bf, device=dev),
                  torch.zeros((1, cfg.n_kv, max_len, cfg.head_dim), dtype=bf, device=dev)) for _ in range(na)],
          "conv": [torch.zeros((1, 3, CD), dtype=bf, device=dev) for _ in range(nl)],
          "ssm": [torch.zeros((1, HV, DV, DK), device=dev) for _ in range(nl)]}
    pc = qt.prefix_cache.PrefixCache(budget_mb=4096)
    node = pc.insert(None, np.arange(pos, dtype=np.int32), pos, st)
    t1 = time_graph(torch, lambda: pc._snapshot(st, 0, pos), reps=40, inner=4)
    t2 = time_graph(torch, lambda: pc.restore(node, max_len), reps=40, inner=4)
    moved = na * 2 * cfg.n_kv * pos * cfg.head_dim * 2 + nl * (HV * DV * DK * 4 + 3 * CD * 2)
    pad = na * 2 * cfg.n_kv * (max_len - pos) * cfg.head_dim * 2
    return {"pos": pos, "max_len": max_len, "checkpoint_us": t1 * 1e6, "checkpoint_GBps": 2 * moved / t1 / 1e9,
            "restore_us": t2 * 1e6, "restore_GBps": (2 * moved + pad) / t2 / 1e9, "node_bytes": node.nbytes}


def cpu_baseline(B, budget_s=12.0):
    """The C restatement of the reference arithmetic (oracle/gdn_oracle.c) timed on this host's cores: a reported baseline only,
    not the reference's own MLX CPU backend (its op-by-op fallback is not part of the reference).  Two legs: config 1's batched
    decode step (the headline's unit, steps/s) and config 0 (one layer, B=1, T=256, token by token; the loop of the
    reference's bench/gdn_f64.py:48-56)."""
    import numpy as np
    from oracle import c_oracle as C
    host = os.cpu_count() or 1
    threads = min(16, host)
    rng = np.random.default_rng(0)
    as_bf = lambda a: (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)
    proj = as_bf(rng.standard_normal((B, PW)))
    conv = as_bf(rng.standard_normal(((B + 1) * 2, 3, CD)))
    cw = as_bf(rng.standard_normal(CD * 4) * 0.5)
    ssm = (rng.standard_normal((B + 1, HV, DV, DK)) * 0.02).astype(np.float32)
    A_log = rng.uniform(0, 2.7, HV).astype(np.float32)
    dtb = (rng.standard_normal(HV) * 0.1).astype(np.float32)
    slots = rng.permutation(B).astype(np.int32)
    pos = np.zeros(B, np.int32)
    C.decode_step(proj, conv, cw, A_log, dtb, ssm, slots, pos, acc64=False, nthreads=threads)      # warm-up
    n, t0 = 0, time.perf_counter()
    while True:
        C.decode_step(proj, conv, cw, A_log, dtb, ssm, slots, pos + n + 1, acc64=False, nthreads=threads)
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s or n >= 20000:
            break
    out = {"value": n / el, "unit": "steps/s", "cores": threads, "host_cores": host, "kind": "port",
           "sample": f"{n} decode steps at B={B} on one layer pool, C restatement of the reference step (oracle/gdn_oracle.c), "
                     f"float accumulation, OpenMP over (row, head) on {threads} threads, {el:.1f} s"}

    # config 0: q, k normalised, v ~ N(0,1), beta = sigmoid(N(0,1)), g from A_log / dt_bias, state from zero; one call per token
    T = 256
    unit = lambda x: x / np.sqrt((x * x).sum(-1, keepdims=True))
    q = as_bf(unit(rng.standard_normal((1, T, HV, DK))) / np.sqrt(DK))
    k = as_bf(unit(rng.standard_normal((1, T, HV, DK))))
    v = as_bf(rng.standard_normal((1, T, HV, DV)))
    beta = as_bf(1.0 / (1.0 + np.exp(-rng.standard_normal((1, T, HV)))))
    sp = np.log1p(np.exp(rng.standard_normal((1, T, HV)) + dtb))
    g = np.exp(-np.exp(A_log) * sp).astype(np.float32)
    tok = lambda a, t: np.ascontiguousarray(a[:, t:t + 1])

    def run_tokens(nthreads):
        st = np.zeros((1, HV, DV, DK), np.float32)
        t0 = time.perf_counter()
        for t in range(T):
            C.recurrent(tok(q, t), tok(k, t), tok(v, t), tok(g, t), tok(beta, t), st, acc64=True, nthreads=nthreads)
        return time.perf_counter() - t0
    run_tokens(threads)
    best = {}
    for nt in sorted({1, threads}):
        reps, t_acc = 0, []
        while sum(t_acc) < budget_s / 4 and reps < 50:
            t_acc.append(run_tokens(nt))
            reps += 1
        t_acc.sort()
        best[nt] = (t_acc[len(t_acc) // 2], reps)
    nt = min(best, key=lambda c: best[c][0])
    out["config0"] = {"value": T / best[nt][0], "unit": "tok/s", "cores": nt, "host_cores": host, "kind": "port",
                      "ms_per_256_tokens": best[nt][0] * 1e3,
                      "sample": f"one GatedDeltaNet layer, B=1, T={T}, one call of the C recurrence (float64 dot products) per token, "
                                f"median of {best[nt][1]} runs; " + ", ".join(f"{c} thread(s): {T / best[c][0]:.0f} tok/s" for c in sorted(best))}
    return out


def profile_leg(torch, qt, dev, args):
    """Runs one leg eagerly a few times so that rocprofv3 (--kernel-trace --stats, or --pmc) sees a short, clean trace."""
    leg, n = args.only, max(1, min(args.steps, 72))
    if leg == "decode":
        st = build_decode_state(torch, dev, args.batch, N_LAYERS)
        for i in range(n):
            l = i % N_LAYERS
            qt.batch.deltanet_b(st["proj"][l & 3], st["conv"][l], st["cw"][l], st["A_log"][l], st["dtb"][l], st["ssm"][l], st["slots"],
                                st["pos"][(i // N_LAYERS) & 1])
    elif leg == "decode_graph":
        # the headline's launch form: HIP graphs of 18 launches (one per layer pool), replayed
        st = build_decode_state(torch, dev, args.batch, N_LAYERS)
        time_decode(torch, qt, st, args.batch, N_LAYERS, 18 * max(1, n // 18), 36, use_graph=True, min_total_s=0.0, max_regions=3)
    elif leg == "copy":
        # plain copy of known size: the scale factor for the FETCH_SIZE / WRITE_SIZE counters (64 MiB read + 64 MiB written)
        src = [torch.randn(16 * 1024 * 1024, device=dev) for _ in range(N_LAYERS)]
        dst = [torch.empty_like(src[0]) for _ in range(2)]
        for i in range(n):
            dst[i & 1].copy_(src[i % N_LAYERS])
    elif leg == "prefill":
        bench_prefill_once(torch, qt, dev, 2048, calls=20)
    elif leg == "prefill_long":
        bench_prefill_once(torch, qt, dev, 8192, calls=10)
    elif leg == "verify":
        bench_verify_gdn(torch, qt, dev)
    elif leg == "attn_decode":
        bench_attn(torch, qt, dev, 16, 1, 512, 32768, 1003)
    elif leg == "attn_verify":
        bench_attn(torch, qt, dev, 16, 4, 1024, 8192, 1004)
    elif leg == "attn_layer":
        bench_attn_layer(torch, qt, dev, 16, 4, 1024, 8192, 1004)
    elif leg == "attn_prefill":
        bench_attn_prefill(torch, qt, dev)
    elif leg == "projections":
        bench_projections(torch, qt, dev)
    elif leg == "state_admission":
        bench_state_admission(torch, qt, dev)
    elif leg == "prefix_cache":
        bench_prefix_cache(torch, qt, dev)
    elif leg == "attn_glue":
        bench_attn_glue(torch, qt, dev)
    elif leg == "attn_prefill_long":
        bench_attn_prefill(torch, qt, dev, 8192)
    else:
        raise SystemExit(f"unknown leg {leg}")
    torch.cuda.synchronize()
    print(json.dumps({"profiled": leg, "launches": n}))


def bench_prefill_once(torch, qt, dev, T, seed=1002, calls=15):
    """the layer core over T tokens, launched eagerly `calls` times on input sets that rotate past the last-level cache"""
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    n_sets = max(8, -(-(LLC_BYTES + LLC_BYTES // 4) // (T * PW * 2)))
    base = torch.randn((T, PW), generator=g).to(bf)
    sets = [(torch.roll(base, shifts=i * 37, dims=0).to(dev), torch.randn((1, 3, CD), generator=g).to(bf).to(dev),
             (torch.randn((1, HV, DV, DK), generator=g) * 0.02).to(dev)) for i in range(n_sets)]
    cw = (torch.randn((CD, 4), generator=g) * 0.5).to(bf).to(dev)
    A, dtb = (torch.rand(HV, generator=g) * 2.7).to(dev), (torch.randn(HV, generator=g) * 0.1).to(dev)
    gw = torch.ones(DV, device=dev)
    for i in range(calls):
        proj, cs, S0 = sets[i % n_sets]
        qt.prefill.gdn_core(proj, cs, S0, cw, A, dtb, gw)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3600)
    ap.add_argument("--warmup", type=int, default=360)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-graph", action="store_true", help="launch every step eagerly instead of replaying HIP graphs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the B sweep and the single-pool run")
    ap.add_argument("--only", default="", help="profile helper: run only one leg a few times and exit "
                                               "(decode | decode_graph | copy | prefill | prefill_long | verify | attn_decode | attn_verify | attn_layer | attn_prefill | attn_prefill_long | "
                                               "projections | state_admission | prefix_cache | attn_glue)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every work item of the path is an independent (slot, head) pair; "
              "there is no multi-GPU leg to time).  Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import qwen_tailor_amd as qt
    qt._lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B = args.batch

    if args.only:
        return profile_leg(torch, qt, dev, args)

    st = build_decode_state(torch, dev, B, N_LAYERS)
    wall, dev_s, n_regions = time_decode(torch, qt, st, B, N_LAYERS, args.steps, args.warmup, use_graph=not args.no_graph)
    # Two clocks around the same regions.  `value` and `ms_per_step` are on the host's wall clock (device synchronisation on both
    # sides of exactly `steps` launches: what a caller waits for); the roofline is on
    # the device clock (HIP events on the launching stream), which leaves out the bracket's own cost.
    launch_s = dev_s / args.steps
    wall_step_s = wall / args.steps
    steps_per_s = 1.0 / wall_step_s
    achieved = decode_bytes(B) / launch_s / 1e9

    extras = {}
    if not args.no_extras:
        # the serving step of one layer: decode step + gated RMSNorm, as two launches and as the fused launch
        gw = torch.ones(DV, device=dev)
        it = [0]

        def two():
            l = it[0] % N_LAYERS
            it[0] += 1
            y = qt.batch.deltanet_b(st["proj"][l & 3], st["conv"][l], st["cw"][l], st["A_log"][l], st["dtb"][l], st["ssm"][l], st["slots"],
                                    st["pos"][0])
            qt.batch.gnorm_rows(y, st["proj"][l & 3], gw)

        def one():
            l = it[0] % N_LAYERS
            it[0] += 1
            qt.batch.deltanet_b_gnorm(st["proj"][l & 3], st["conv"][l], st["cw"][l], st["A_log"][l], st["dtb"][l], st["ssm"][l], st["slots"],
                                      st["pos"][0], gw)
        t2 = time_graph(torch, two, reps=N_LAYERS * 20, inner=N_LAYERS)
        t1 = time_graph(torch, one, reps=N_LAYERS * 20, inner=N_LAYERS)
        extras["decode_plus_gated_norm"] = {"two_launches_us": t2 * 1e6, "fused_us": t1 * 1e6,
                                            "fused_GBps": (decode_bytes(B) + B * 2048 * 2) / t1 / 1e9}
        # the whole GatedDeltaNet half of a layer at a decode step (qwen35/batch.py:496-501): rms_rows, in_proj, the step with
        # the gated norm, out_proj with the residual: four launches
        g = torch.Generator().manual_seed(3)
        bf = torch.bfloat16
        Wi = [(torch.randn((PW, 1024), generator=g) / 32).to(bf).to(dev) for _ in range(8)]
        Wo = [(torch.randn((1024, 2048), generator=g) / 45).to(bf).to(dev) for _ in range(8)]
        xh = torch.randn((B, 1024), generator=g).to(bf).to(dev)
        ln = torch.ones(1024, dtype=bf, device=dev)

        def layer():
            l = it[0] % N_LAYERS
            it[0] += 1
            proj = qt.kernels.fused_gemv(Wi[l & 7], qt.batch.rms_rows(xh, ln))
            yn = qt.batch.deltanet_b_gnorm(proj, st["conv"][l], st["cw"][l], st["A_log"][l], st["dtb"][l], st["ssm"][l], st["slots"],
                                           st["pos"][0], gw)
            qt.kernels.fused_gemv(Wo[l & 7], yn, res=xh)
        t3 = time_graph(torch, layer, reps=N_LAYERS * 10, inner=N_LAYERS)
        extras["gdn_layer_half_decode"] = {"B": B, "launches": 4, "us": t3 * 1e6}
        del Wi, Wo
        w1, d1, _ = time_decode(torch, qt, st, B, 1, args.steps, args.warmup, use_graph=not args.no_graph)
        extras["single_pool_cache_resident"] = {"steps_per_s": args.steps / d1, "wall_steps_per_s": args.steps / w1,
                                                "GBps": decode_bytes(B) / (d1 / args.steps) / 1e9}
        if not args.no_graph:
            w2, d2, _ = time_decode(torch, qt, st, B, N_LAYERS, args.steps, args.warmup, use_graph=False)
            extras["eager_launch"] = {"steps_per_s": args.steps / d2, "wall_steps_per_s": args.steps / w2,
                                      "GBps": decode_bytes(B) / (d2 / args.steps) / 1e9}
        del st
        torch.cuda.empty_cache()
        for b in (1, 16):
            stb = build_decode_state(torch, dev, b, N_LAYERS)
            wb, db, _ = time_decode(torch, qt, stb, b, N_LAYERS, args.steps, args.warmup, use_graph=not args.no_graph)
            extras[f"B{b}"] = {"steps_per_s": args.steps / db, "wall_steps_per_s": args.steps / wb, "us_per_step": db / args.steps * 1e6,
                               "GBps": decode_bytes(b) / (db / args.steps) / 1e9}
            del stb
        torch.cuda.empty_cache()
        extras["gdn_prefill"] = [bench_prefill(torch, qt, dev, T) for T in (512, 2048, 8192)]
        extras["gdn_verify"] = bench_verify_gdn(torch, qt, dev)
        extras["attn_decode_config3"] = bench_attn(torch, qt, dev, 16, 1, 512, 32768, 1003)
        torch.cuda.empty_cache()
        extras["attn_verify_config4"] = bench_attn(torch, qt, dev, 16, 4, 1024, 8192, 1004)
        extras["attn_layer_half_config4"] = bench_attn_layer(torch, qt, dev, 16, 4, 1024, 8192, 1004)
        torch.cuda.empty_cache()
        extras["attn_layer_half_config3"] = bench_attn_layer(torch, qt, dev, 16, 1, 512, 32768, 1003)
        torch.cuda.empty_cache()
        extras["attn_prefill_causal"] = [bench_attn_prefill(torch, qt, dev, S) for S in (2048, 8192)]
        extras["state_admission"] = bench_state_admission(torch, qt, dev)
        extras["attn_glue"] = bench_attn_glue(torch, qt, dev)
        extras["gdn_layer_projections"] = bench_projections(torch, qt, dev)
        extras["prefix_cache"] = bench_prefix_cache(torch, qt, dev)

    out = {
        "metric": "GDN decode steps/s @B=64 (% HBM peak); GDN prefill tok/s @2048 (% MFMA)",
        "value": steps_per_s, "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_step_s * 1e3, "clock": "host wall clock, device synchronised on both sides of each region",
        "value_device_clock": 1.0 / launch_s, "ms_per_step_device_clock": launch_s * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"configs[1]: batched GDN decode step, B={B} slots, 16 heads x 128x128 fp32 state per slot, "
                               f"rotating over {N_LAYERS} layer pools", "batch": B, "layer_pools": N_LAYERS,
                   "launch": "eager" if args.no_graph else "hip-graph of 18 launches",
                   "timing": f"median of {n_regions} regions of {args.steps} launches; value on the host wall clock, roofline on HIP "
                             f"events on the launching stream around the same regions"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": DECODE_TRAFFIC_B64 if B == 64 else None,
                     "traffic_source": DECODE_TRAFFIC_SOURCE if B == 64 else None,
                     "kernel": "gdn_decode_wide_kernel<4>" if B >= 64 else "gdn_decode_kernel", "bytes_per_launch": decode_bytes(B),
                     "avg_launch_us": launch_s * 1e6, "clock": "HIP events on the launching stream",
                     "frac_on_wall_clock": decode_bytes(B) / wall_step_s / 1e9 / HBM_PEAK_GBS},
        "extras": extras,
    }
    if "gdn_prefill" in extras:
        p2k = extras["gdn_prefill"][1]
        out["secondary"] = {"metric": "GDN prefill tok/s @2048 (% MFMA)", "value": p2k["tok_per_s"], "unit": "tok/s",
                            "config": {"workload": "configs[2]: conv + chunked GDN (chunk 64) + gated RMSNorm, B=1, T=2048, 16 heads, "
                                                   "nonzero initial state"},
                            "roofline": {"bound": "mfma", "achieved": p2k["mfma_tflops"], "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                                         "frac": p2k["mfma_frac"], "traffic": PREFILL_TRAFFIC_T2048,
                                         "traffic_source": PREFILL_TRAFFIC_SOURCE}}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(B)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
