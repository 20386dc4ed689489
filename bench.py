#!/usr/bin/env python3
"""Benchmark of the MI355X Muon / Dion optimizer-step hot path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A "step" is one full optimizer step over every matrix of the workload with synthetic
Gaussian gradients already resident in HBM.  Prints ONE JSON line.

Workloads (BASELINE.json `configs`):
  muon_gpt_small   (default) full Muon step, GPT-small: 72 bf16 matrices (48 x 768^2,
                   12 x 3072x768, 12 x 768x3072), G ~ N(0,1e-3) seed 1, mu 0.95 Nesterov.
  muon_llama8b_layer   Muon NS5 on one Llama-3-8B layer's matrices (bf16), seed 4.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_FLOPS = 2.5e15   # MI355X dense bf16 MFMA
PEAK_HBM_BPS = 8.0e12      # MI355X HBM3E

GPT_SMALL_LAYER = [(768, 768)] * 4 + [(3072, 768), (768, 3072)]
LLAMA8B_LAYER = [(4096, 4096)] * 2 + [(1024, 4096)] * 2 + [(14336, 4096)] * 2 + [(4096, 14336)]

WORKLOADS = {
    "muon_gpt_small": dict(shapes=GPT_SMALL_LAYER * 12, seed=1,
                           desc="Full Muon step, GPT-small (12 layers, d=768): 72 bf16 matrices"),
    "muon_llama8b_layer": dict(shapes=LLAMA8B_LAYER, seed=4,
                               desc="Muon step, one Llama-3-8B layer: 7 bf16 matrices incl. 4096x14336"),
}


def make_problem(shapes, seed, device, dtype):
    import torch

    gen = torch.Generator(device="cpu").manual_seed(seed)
    params, grads = [], []
    for s in shapes:
        w = (torch.randn(s, generator=gen) * 0.02).to(dtype)
        g = (torch.randn(s, generator=gen) * 1e-3).to(dtype)
        params.append(w)
        grads.append(g)
    return params, grads


def ns_flops(shapes, symmetric):
    tot = 0
    for m, n in shapes:
        mw, nw = min(m, n), max(m, n)
        tot += 5 * ((3 * mw * mw * nw + mw**3) if symmetric else (4 * mw * mw * nw + 2 * mw**3))
    return tot


def cpu_baseline(shapes, seed, budget_s=20.0):
    """The oracle (eager-PyTorch CPU restatement of the reference step) timed on the host cores."""
    import torch
    from oracle import muon_step as O

    X, G = make_problem(shapes, seed, "cpu", torch.bfloat16)
    M = [torch.zeros_like(x) for x in X]
    t0 = time.perf_counter()
    O.muon_step(X, G, M, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True)  # warm-up
    first = time.perf_counter() - t0
    reps = max(1, min(10, int(budget_s / max(first, 1e-3)) - 1))
    t0 = time.perf_counter()
    for _ in range(reps):
        O.muon_step(X, G, M, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True)
    ms = (time.perf_counter() - t0) / reps * 1e3
    return dict(value=round(ms, 3), unit="ms", cores=torch.get_num_threads(), kind="port",
                sample=f"{reps} full steps of the same {len(shapes)}-matrix workload after 1 warm-up "
                       f"(eager PyTorch CPU, bf16, Nesterov)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="muon_gpt_small", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from dion_amd import Muon, _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    wl = WORKLOADS[args.workload]
    shapes = wl["shapes"]
    X, G = make_problem(shapes, wl["seed"], dev, torch.bfloat16)
    params = [torch.nn.Parameter(x.to(dev)) for x in X]
    for p, g in zip(params, G):
        p.grad = g.to(dev)
    opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, adjust_lr="spectral_norm")

    for _ in range(args.warmup):
        opt.step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        opt.step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = e0.elapsed_time(e1) / args.steps
    ms_per_step = max(wall_ms, ev_ms)

    # per-kernel HIP-event timing of the same steps (events bracket every launch on its stream)
    lib = _lib.load()
    lib.dion_amd_profile_reset()
    lib.dion_amd_profile_enable(1)
    for _ in range(args.steps):
        opt.step()
    torch.cuda.synchronize()
    lib.dion_amd_profile_enable(0)
    prof = _lib.profile_read()
    lib.dion_amd_profile_reset()

    kernels = {}
    for name, (n, ms, work) in prof.items():
        is_gemm = name.startswith("ns_") or name in ("gemm", "dion_bq", "dion_btp", "dion_ef", "dion_upd")
        rate = work / (ms * 1e-3) if ms > 0 else 0.0
        kernels[name] = dict(launches_per_step=n / args.steps, avg_ms=ms / n, ms_per_step=ms / args.steps,
                             **({"tflops": rate / 1e12, "frac_mfma": rate / PEAK_BF16_FLOPS} if is_gemm
                                else {"gbps": rate / 1e9, "frac_hbm": rate / PEAK_HBM_BPS}))
    gemm_kinds = [k for k in ("ns_syrk", "ns_poly", "ns_axpy") if k in prof]
    dom = max(gemm_kinds, key=lambda k: prof[k][1])
    n, ms, work = prof[dom]
    achieved = work / (ms * 1e-3) / 1e12
    roofline = dict(bound="mfma", kernel=dom, achieved=round(achieved, 2), peak=PEAK_BF16_FLOPS / 1e12,
                    unit="TFLOP/s", frac=round(achieved * 1e12 / PEAK_BF16_FLOPS, 4), traffic=None,
                    avg_launch_ms=round(ms / n, 5),
                    flops_per_launch=work / n)
    ns_ms = sum(prof[k][1] for k in gemm_kinds) / args.steps
    f_sym = ns_flops(shapes, True)

    out = {
        "metric": "Muon/Dion optimizer-step ms (GPT-160M, 8B-layer) + % bf16 MFMA peak",
        "value": round(ms_per_step, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": wl["desc"], "matrices": len(shapes),
                   "optimizer": "Muon(lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01, adjust_lr=spectral_norm)",
                   "grad": f"N(0,1e-3) seed {wl['seed']}", "parallelism": "single GPU"},
        "orthogonalisations_per_s": round(len(shapes) / (ms_per_step * 1e-3), 1),
        "ns_gemm_ms_per_step": round(ns_ms, 4),
        "ns_executed_tflops": round(f_sym / (ns_ms * 1e-3) / 1e12, 2) if ns_ms > 0 else None,
        "ns_frac_mfma_peak": round(f_sym / (ns_ms * 1e-3) / PEAK_BF16_FLOPS, 4) if ns_ms > 0 else None,
        "ns_dense_convention_tflops": round(ns_flops(shapes, False) / (ns_ms * 1e-3) / 1e12, 2) if ns_ms > 0 else None,
        "event_ms_per_step": round(ev_ms, 4),
        "wall_ms_per_step": round(wall_ms, 4),
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(shapes, wl["seed"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
