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


def time_decode(torch, qt, st, B, n_layers, steps, warmup, use_graph=True):
    """Times exactly `steps` launches after `warmup` untimed ones.  Returns (wall seconds, device seconds from events)."""
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

    i = run(warmup)
    i = ((i + n_layers - 1) // n_layers) * n_layers if graphs is not None else i
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    run(steps, i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) * 1e-3


def cpu_baseline(B, budget_s=12.0):
    """The C restatement of the decode step (float accumulation) timed on this host's cores: a reported baseline only."""
    import numpy as np
    from oracle import c_oracle as C
    threads = min(16, os.cpu_count() or 1)
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
        if el >= budget_s or n >= 5000:
            break
    return {"value": n / el, "unit": "steps/s", "cores": threads, "kind": "port",
            "sample": f"{n} decode steps at B={B} on one layer pool, C restatement of the reference step (oracle/gdn_oracle.c), "
                      f"float accumulation, OpenMP over (row, head), {el:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3600)
    ap.add_argument("--warmup", type=int, default=360)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-graph", action="store_true", help="launch every step eagerly instead of replaying HIP graphs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the B sweep and the single-pool run")
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

    st = build_decode_state(torch, dev, B, N_LAYERS)
    wall, dev_s = time_decode(torch, qt, st, B, N_LAYERS, args.steps, args.warmup, use_graph=not args.no_graph)
    steps_per_s = args.steps / wall
    launch_s = dev_s / args.steps
    achieved = decode_bytes(B) / launch_s / 1e9

    extras = {}
    if not args.no_extras:
        w1, d1 = time_decode(torch, qt, st, B, 1, args.steps, args.warmup, use_graph=not args.no_graph)
        extras["single_pool_cache_resident"] = {"steps_per_s": args.steps / w1, "GBps": decode_bytes(B) / (d1 / args.steps) / 1e9}
        if not args.no_graph:
            w2, d2 = time_decode(torch, qt, st, B, N_LAYERS, args.steps, args.warmup, use_graph=False)
            extras["eager_launch"] = {"steps_per_s": args.steps / w2, "GBps": decode_bytes(B) / (d2 / args.steps) / 1e9}
        del st
        torch.cuda.empty_cache()
        for b in (1, 16):
            stb = build_decode_state(torch, dev, b, N_LAYERS)
            wb, db = time_decode(torch, qt, stb, b, N_LAYERS, args.steps, args.warmup, use_graph=not args.no_graph)
            extras[f"B{b}"] = {"steps_per_s": args.steps / wb, "us_per_step": db / args.steps * 1e6,
                               "GBps": decode_bytes(b) / (db / args.steps) / 1e9}
            del stb

    out = {
        "metric": "GDN decode steps/s @B=64 (% HBM peak); GDN prefill tok/s @2048 (% MFMA)",
        "value": steps_per_s, "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"configs[1]: batched GDN decode step, B={B} slots, 16 heads x 128x128 fp32 state per slot, "
                               f"rotating over {N_LAYERS} layer pools", "batch": B, "layer_pools": N_LAYERS,
                   "launch": "eager" if args.no_graph else "hip-graph of 18 launches"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": None, "kernel": "gdn_decode_kernel<8>", "bytes_per_launch": decode_bytes(B),
                     "avg_launch_us": launch_s * 1e6},
        "extras": extras,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(B)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
