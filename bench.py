#!/usr/bin/env python3
"""Benchmark of the MI355X Muon / Dion optimizer-step hot path (one GPU).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--no-cpu-baseline]

A "step" is one full optimizer step over every matrix of the workload, with synthetic
Gaussian gradients already resident in HBM.  Prints ONE JSON line whose `value` is the
milliseconds per step of the selected workload; the other benchmark configurations that fit
in a short run are reported under `extra`.

Workloads (numbered as the benchmark's configurations):
  muon_gpt_small        (default, configs[1]) full Muon step, GPT-small: 72 bf16 matrices
                        (48 x 768^2, 12 x 3072x768, 12 x 768x3072), G ~ N(0,1e-3) seed 1, Nesterov.
  dion_gpt_small_r025   (configs[2]) full Dion step on the same matrices, rank fraction 0.25,
  dion_gpt_small_r1     rank fraction 1.0; bf16 weights / momentum, fp32 Q, G seed 3.
  muon_llama8b_layer    (configs[3], one of the 32 layers) Muon on 7 bf16 matrices incl. 4096x14336.
  muon_4096x14336       one bucket of 32 matrices of 4096x14336 (W_down of the 32 layers): the shape the
                        Newton-Schulz target is quoted on, per-product fractions of the bf16 peak.
  dion_llama70b_layer   (configs[4], one of the 8 layers) Dion r=512 on 2 x 28672x8192 + 8192x28672.
  muon_llama8b          (configs[3], all 32 layers) 224 bf16 matrices, 6.98e9 elements, drawn on the GPU.
  dion_llama70b_mlp     (configs[4], all 8 layers) 24 bf16 matrices, 5.64e9 elements, drawn on the GPU.
  scalar_gpt_small      the non-matrix groups of GPT-small: Lion / AdamW on embedding, lm_head, norms.
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
LLAMA70B_MLP_LAYER = [(28672, 8192)] * 2 + [(8192, 28672)]

WORKLOADS = {
    "muon_gpt_small": dict(kind="muon", shapes=GPT_SMALL_LAYER * 12, seed=1, graph=True,
                           desc="Full Muon step, GPT-small (12 layers, d=768): 72 bf16 matrices"),
    "dion_gpt_small_r025": dict(kind="dion", shapes=GPT_SMALL_LAYER * 12, seed=3, rank_fraction=0.25, graph=True,
                                desc="Full Dion step, GPT-small matrices, rank fraction 0.25 (r=192), bf16 M, fp32 Q"),
    "dion_gpt_small_r1": dict(kind="dion", shapes=GPT_SMALL_LAYER * 12, seed=3, rank_fraction=1.0, graph=True,
                              desc="Full Dion step, GPT-small matrices, rank fraction 1.0 (r=768), bf16 M, fp32 Q"),
    "muon_llama8b_layer": dict(kind="muon", shapes=LLAMA8B_LAYER, seed=4,
                               desc="Muon step, one Llama-3-8B layer: 7 bf16 matrices incl. 4096x14336"),
    "dion_llama70b_layer": dict(kind="dion", shapes=LLAMA70B_MLP_LAYER, seed=5, rank_fraction=1.0 / 16,
                                desc="Dion step, one Llama-3-70B MLP layer (28672x8192 x2, 8192x28672), r=512"),
    "muon_4096x14336": dict(kind="muon", shapes=[(4096, 14336)] * 32, seed=4, on_device=True,
                            desc="Muon step on the bucket of 32 4096x14336 bf16 matrices (W_down of a Llama-3-8B stack): "
                                 "the shape the 60 % target names"),
    "muon_llama8b": dict(kind="muon", shapes=LLAMA8B_LAYER * 32, seed=4, on_device=True,
                         desc="Full Muon step, Llama-3-8B-shaped stack: 32 layers x 7 bf16 matrices (6.98e9 elements)"),
    "dion_llama70b_mlp": dict(kind="dion", shapes=LLAMA70B_MLP_LAYER * 8, seed=5, rank_fraction=1.0 / 16, on_device=True,
                              desc="Full Dion step, Llama-3-70B-shaped MLP matrices: 8 layers x 3 (5.64e9 elements), r=512"),
    "scalar_gpt_small": dict(kind="scalar", shapes=[(50304, 768)] * 2 + [(768,)] * 25, seed=6,
                             desc="Lion on the GPT-small embedding and norms, AdamW on lm_head (50304x768 each), bf16"),
}
GEMM_KINDS = ("ns_syrk", "ns_poly", "ns_axpy", "ns_flow", "gemm", "dion_bq", "dion_btp", "dion_ef", "dion_upd", "dion_ef_upd")


def make_problem(shapes, seed, dtype, device="cpu"):
    """Weights N(0, 0.02^2) and gradients N(0, 1e-6) from a seeded generator; the multi-gigabyte workloads draw
    them on the GPU (the values differ from the CPU generator's, the distribution does not)."""
    import torch

    gen = torch.Generator(device=device).manual_seed(seed)
    params, grads = [], []
    for s in shapes:
        params.append((torch.randn(s, generator=gen, device=device) * 0.02).to(dtype))
        grads.append((torch.randn(s, generator=gen, device=device) * 1e-3).to(dtype))
    return params, grads


def ns_flops(shapes, symmetric):
    tot = 0
    for m, n in shapes:
        mw, nw = min(m, n), max(m, n)
        tot += 5 * ((3 * mw * mw * nw + mw**3) if symmetric else (4 * mw * mw * nw + 2 * mw**3))
    return tot


def build_optimizer(wl, dev):
    import torch
    from dion_amd import Dion, DionMixedPrecisionConfig, Muon

    X, G = make_problem(wl["shapes"], wl["seed"], torch.bfloat16, dev if wl.get("on_device") else "cpu")
    params = [torch.nn.Parameter(x.to(dev)) for x in X]
    for p, g in zip(params, G):
        p.grad = g.to(dev)
    if wl["kind"] == "scalar":
        opt = Muon([dict(params=[params[0]] + params[2:], algorithm="lion"),
                    dict(params=[params[1]], algorithm="adamw")], lr=0.01, weight_decay=0.01)
        desc = "Muon(param groups: lion [embedding, 25 norm vectors], adamw [lm_head]; lr=0.01, betas=(0.9, 0.95), wd=0.01)"
        return opt, params, desc
    if wl["kind"] == "muon":
        opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, adjust_lr="spectral_norm")
        desc = "Muon(lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01, adjust_lr=spectral_norm)"
    else:
        torch.manual_seed(2)
        opt = Dion(params, rank_fraction=wl["rank_fraction"], lr=0.01, mu=0.95, weight_decay=0.01,
                   mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=torch.bfloat16, Q_dtype=torch.float32))
        desc = (f"Dion(rank_fraction={wl['rank_fraction']:.4g}, lr=0.01, mu=0.95, weight_decay=0.01, "
                "momentum bf16, Q fp32)")
    return opt, params, desc


def measure(wl, dev, steps, warmup):
    """Timed region + a second pass of the same steps with per-launch HIP events."""
    import torch
    from dion_amd import _lib

    opt, params, desc = build_optimizer(wl, dev)
    for _ in range(warmup):
        opt.step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        opt.step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = e0.elapsed_time(e1) / steps

    # The same step captured once in a HIP graph and replayed (no per-launch host work): what a training loop that
    # captures its optimizer step gets.  Only for the workloads whose step is short enough to be bound by the host.
    graph_ms = None
    if wl.get("graph"):
        try:
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    opt.step()
            torch.cuda.synchronize()
            for _ in range(warmup):
                graph.replay()
            torch.cuda.synchronize()
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            tg = time.perf_counter()
            g0.record()
            for _ in range(steps):
                graph.replay()
            g1.record()
            torch.cuda.synchronize()
            graph_ms = max((time.perf_counter() - tg) * 1e3 / steps, g0.elapsed_time(g1) / steps)
            del graph
        except Exception as exc:   # the figure is an extra: the run goes on without it
            graph_ms = f"capture failed: {exc}"

    # Second pass for the per-launch figures.  Dion runs its buckets on up to three streams; for this
    # pass they run one at a time so that a launch's duration is that of the kernel alone.
    if hasattr(opt, "_max_concurrent_tasks"):
        opt._max_concurrent_tasks = 1
    lib = _lib.load()
    lib.dion_amd_profile_reset()
    lib.dion_amd_profile_enable(1)
    for _ in range(steps):
        opt.step()
    torch.cuda.synchronize()
    lib.dion_amd_profile_enable(0)
    prof = _lib.profile_read()
    lib.dion_amd_profile_reset()

    kernels = {}
    for name, (n, ms, work) in prof.items():
        rate = work / (ms * 1e-3) if ms > 0 else 0.0
        k = dict(launches_per_step=round(n / steps, 2), avg_ms=round(ms / n, 5), ms_per_step=round(ms / steps, 4))
        if name in GEMM_KINDS:
            k.update(tflops=round(rate / 1e12, 1), frac_mfma=round(rate / PEAK_BF16_FLOPS, 4))
        elif work > 0:
            k.update(gbps=round(rate / 1e9, 1), frac_hbm=round(rate / PEAK_HBM_BPS, 4))
        kernels[name] = k
    res = dict(ms_per_step=max(wall_ms, ev_ms), wall_ms=wall_ms, event_ms=ev_ms, kernels=kernels, prof=prof,
               optimizer=desc, steps=steps, graph_ms=graph_ms)
    del opt, params
    torch.cuda.empty_cache()
    return res


def summarize(name, wl, res):
    shapes = wl["shapes"]
    out = dict(workload=name, ms_per_step=round(res["ms_per_step"], 4), steps=res["steps"],
               orthogonalisations_per_s=round(len(shapes) / (res["ms_per_step"] * 1e-3), 1))
    if res.get("graph_ms") is not None:
        g = res["graph_ms"]
        out["hip_graph_replay_ms_per_step"] = round(g, 4) if isinstance(g, float) else g
    prof = res["prof"]
    if wl["kind"] == "muon":
        ns_ms = sum(prof[k][1] for k in ("ns_syrk", "ns_poly", "ns_axpy", "ns_flow") if k in prof) / res["steps"]
        f_sym = ns_flops(shapes, True)
        out.update(ns_gemm_ms_per_step=round(ns_ms, 4),
                   ns_executed_tflops=round(f_sym / (ns_ms * 1e-3) / 1e12, 1),
                   ns_frac_mfma_peak=round(f_sym / (ns_ms * 1e-3) / PEAK_BF16_FLOPS, 4),
                   ns_dense_convention_tflops=round(ns_flops(shapes, False) / (ns_ms * 1e-3) / 1e12, 1))
    out["kernels"] = res["kernels"]
    if wl["kind"] == "dion":
        # Dion's products sit near the machine balance (arithmetic intensity ~ r flop/byte): report them against
        # the HBM roofline as well.  Algorithmic bytes per step over all matrices, bf16 momentum / weights,
        # factors in the momentum dtype: P = BQ and R = B^T P read B once; the error-feedback and weight-update
        # products read and write an m x n matrix; each also moves its m' x r and n' x r factors.
        import math

        from collections import Counter

        from dion_amd import _lib
        lib = _lib.load()
        rd = bq = upd = fused = 0.0
        for (m, n), count in Counter(shapes).items():
            r = min(math.ceil(wl["rank_fraction"] * min(m, n)), m, n)   # reference dion/dion.py:672-676
            # P = BQ with B = M + G formed inside it also reads G and writes M (the separate pass's bytes are the
            # dion_elem kind's otherwise)
            inside = lib.dion_amd_dion_bq_fused(count, m, n, r, 0, 0)
            bq += count * 2.0 * (m * n * (3 if inside else 1) + (m + n) * r)
        for m, n in shapes:
            r = min(math.ceil(wl["rank_fraction"] * min(m, n)), m, n)
            rd += 2.0 * (m * n + (m + n) * r)
            upd += 2.0 * (2 * m * n + (m + n) * r)
            # error feedback and weight update as one pass: M and X read and written once, P, R and Q_new read
            fused += 2.0 * (4 * m * n + (max(m, n) + 2 * min(m, n)) * r)
        for name, nbytes in (("dion_bq", bq), ("dion_btp", rd), ("dion_ef", upd), ("dion_upd", upd),
                             ("dion_ef_upd", fused)):
            k = out["kernels"].get(name)
            if k and k["ms_per_step"] > 0:
                rate = nbytes / (k["ms_per_step"] * 1e-3)
                k.update(gbps=round(rate / 1e9, 1), frac_hbm=round(rate / PEAK_HBM_BPS, 4))
    return out


# HBM bytes per launch of the dominant kernel, from two `rocprofv3 --pmc` runs (FETCH_SIZE x 2.000 and
# WRITE_SIZE x 1.000, in KiB, the factors being what the same counters read for a plain 512 MiB copy);
# the runs used the workload named in the key with three 512 MiB copies first (--calibrate-copy).  Keyed by
# (workload, kernel); measured 2026-11-25 on the kernels of this revision (profiles/*_hbm_traffic.md hold the runs);
# a kernel kind that is not listed has not been measured since it last changed and reports null.
MEASURED_TRAFFIC_BYTES = {
    # the persistent Newton-Schulz launch: all 15 products of all 72 matrices
    ("muon_gpt_small", "ns_flow"): 5910473 * 1024,
    # X' = aX + BX over the 32 matrices (mean of the five launches; the last one updates the weights instead of storing X')
    ("muon_4096x14336", "ns_axpy"): 29839601 * 1024,
    # one Llama-3-8B layer: the grouped X' = aX + BX launch over its four buckets
    ("muon_llama8b_layer", "ns_axpy"): 3534072 * 1024,
    # error feedback + weight update in one pass: mean over the buckets of the workload
    ("dion_gpt_small_r025", "dion_ef_upd"): 277687 * 1024,
    ("dion_llama70b_layer", "dion_ef_upd"): 4027315 * 1024,
    # mean over the three buckets (two launches of the non-transposed kernel, one of the transposed one)
    ("dion_gpt_small_r1", "dion_ef_upd"): 446671 * 1024,
    # the 16-matrix and the 8-matrix bucket: mean of the two launches
    ("dion_llama70b_mlp", "dion_ef_upd"): 33113826 * 1024,
    # the grouped X' = aX + BX launch over all 224 matrices
    ("muon_llama8b", "ns_axpy"): 108596291 * 1024,
    # mean of the AdamW launch (lm_head) and the Lion launch (embedding, norms)
    ("scalar_gpt_small", "scalar_opt"): 453078 * 1024,
}


def dion_hbm_bytes(wl):
    """Algorithmic HBM bytes per step of the Dion products over all matrices of the workload (bf16 momentum / weights,
    factors in the momentum dtype) and the rank, keyed by kernel kind."""
    import math

    rd = upd = fused = 0.0
    rank = 0
    for m, n in wl["shapes"]:
        r = min(math.ceil(wl["rank_fraction"] * min(m, n)), m, n)   # reference dion/dion.py:672-676
        rank = max(rank, r)
        rd += 2.0 * (m * n + (m + n) * r)
        upd += 2.0 * (2 * m * n + (m + n) * r)
        fused += 2.0 * (4 * m * n + (max(m, n) + 2 * min(m, n)) * r)
    return {"dion_bq": (rd, rank), "dion_btp": (rd, rank), "dion_ef": (upd, rank), "dion_upd": (upd, rank),
            "dion_ef_upd": (fused, rank)}


def roofline_of(res, kind, workload=None, hbm_bytes=None):
    """Dominant kernel of the run: algorithmic flops (bytes for the HBM-bound passes) per launch / average launch
    duration."""
    prof = res["prof"]
    if kind == "scalar":
        n, ms, work = prof["scalar_opt"]
        achieved = work / (ms * 1e-3) / 1e9
        return dict(bound="hbm", kernel="scalar_opt", achieved=round(achieved, 1), peak=PEAK_HBM_BPS / 1e9, unit="GB/s",
                    frac=round(achieved * 1e9 / PEAK_HBM_BPS, 4),
                    traffic=MEASURED_TRAFFIC_BYTES.get((workload, "scalar_opt")), avg_launch_ms=round(ms / n, 5),
                    bytes_per_launch=work / n)
    cands = [k for k in (("ns_syrk", "ns_poly", "ns_axpy", "ns_flow") if kind == "muon"
                         else ("dion_bq", "dion_btp", "dion_ef", "dion_upd", "dion_ef_upd")) if k in prof]
    dom = max(cands, key=lambda k: prof[k][1])
    n, ms, work = prof[dom]
    if kind == "dion" and hbm_bytes is not None and dom in hbm_bytes:
        # A rank-r product moves m n bytes-ish per 2 m n r flops: below r = 312 flop/byte (2.5 PFLOP/s over 8 TB/s) the HBM
        # roofline binds it -- the low-rank configurations; priced against HBM then (algorithmic bytes per launch).
        nbytes, rank = hbm_bytes[dom]
        if rank < PEAK_BF16_FLOPS / PEAK_HBM_BPS:
            achieved = nbytes / (ms / res["steps"] * 1e-3) / 1e9
            return dict(bound="hbm", kernel=dom, achieved=round(achieved, 1), peak=PEAK_HBM_BPS / 1e9, unit="GB/s",
                        frac=round(achieved * 1e9 / PEAK_HBM_BPS, 4), traffic=MEASURED_TRAFFIC_BYTES.get((workload, dom)),
                        avg_launch_ms=round(ms / n, 5), bytes_per_launch=nbytes * res["steps"] / n,
                        mfma_frac=round(work / (ms * 1e-3) / PEAK_BF16_FLOPS, 4))
    achieved = work / (ms * 1e-3) / 1e12
    return dict(bound="mfma", kernel=dom, achieved=round(achieved, 2), peak=PEAK_BF16_FLOPS / 1e12, unit="TFLOP/s",
                frac=round(achieved * 1e12 / PEAK_BF16_FLOPS, 4),
                traffic=MEASURED_TRAFFIC_BYTES.get((workload, dom)),
                avg_launch_ms=round(ms / n, 5), flops_per_launch=work / n)


def cpu_baseline(wl, budget_s=20.0):
    """The oracle (eager-PyTorch CPU restatement of the reference step) timed on the host cores."""
    import torch

    shapes = wl["shapes"]
    X, G = make_problem(shapes, wl["seed"], torch.bfloat16)
    if wl["kind"] == "scalar":
        from oracle import scalar_opts as O

        M = [torch.zeros_like(x) for x in X]
        V = [torch.zeros_like(X[1])]
        t = torch.tensor
        lion = [0] + list(range(2, len(X)))

        def step():
            O.lion_update_foreach([X[i] for i in lion], [G[i] for i in lion], [M[i] for i in lion],
                                  t(0.01), t(0.9), t(0.95), t(0.01))
            O.adamw_update_foreach([X[1]], [G[1]], [M[1]], V, t(0.01), t(0.9), t(0.95), t(0.01), t(1), t(1e-8))
        what = "eager PyTorch CPU foreach ops, bf16"
    elif wl["kind"] == "muon":
        from oracle import muon_step as O

        M = [torch.zeros_like(x) for x in X]

        def step():
            O.muon_step(X, G, M, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True)
        what = "eager PyTorch CPU, bf16, Nesterov"
    else:
        from oracle import dion_step as O

        torch.manual_seed(2)
        M = [torch.zeros_like(x) for x in X]
        Q = [torch.randn((min(s), O.rank_of(s[0], s[1], wl["rank_fraction"]))) for s in shapes]
        gen = torch.Generator().manual_seed(0)

        def step():
            O.dion_step(X, G, M, Q, lr=0.01, mu=0.95, weight_decay=0.01, generator=gen)
        what = "eager PyTorch CPU, bf16 momentum, fp32 Q, reference orthogonalize rule"
    t0 = time.perf_counter()
    step()  # warm-up
    first = time.perf_counter() - t0
    reps = max(1, min(10, int(budget_s / max(first, 1e-3)) - 1))
    t0 = time.perf_counter()
    for _ in range(reps):
        step()
    ms = (time.perf_counter() - t0) / reps * 1e3
    return dict(value=round(ms, 3), unit="ms", cores=torch.get_num_threads(), kind="port",
                sample=f"{reps} full steps of the same {len(shapes)}-matrix workload after 1 warm-up ({what})")


def device_info(dev):
    """What the rooflines are priced against, as the runtime reports it for the GPU the numbers come from."""
    import torch

    p = torch.cuda.get_device_properties(dev)
    info = dict(name=p.name, compute_units=p.multi_processor_count, hbm_gib=round(p.total_memory / 2**30, 1))
    clock_khz = getattr(p, "clock_rate", None)
    if clock_khz:
        info["max_shader_clock_mhz"] = round(clock_khz / 1e3)
        # dense bf16 MFMA: 4096 flops per clock per CU (a 32x32x16 MFMA, 32768 flops, per SIMD every 32 clocks)
        info["bf16_dense_peak_at_that_clock_tflops"] = round(p.multi_processor_count * 4096 * clock_khz * 1e3 / 1e12, 1)
    info["arch"] = getattr(p, "gcnArchName", "")
    return info


def stream_ceiling(dev):
    """What a plain streaming kernel reaches on this GPU in this run (an in-place scale by torch: one read and one
    write per element), at the size of one GPT-small bucket and at 2 GiB: the practical ceiling next to the 8 TB/s
    the HBM-bound passes are priced against."""
    import torch

    out = {}
    for label, n in (("108MiB", 48 * 768 * 768 * 2), ("2GiB", 1 << 30)):
        x = torch.ones(n, dtype=torch.bfloat16, device=dev)
        for _ in range(3):
            x.mul_(1.0)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            x.mul_(1.0)
        e1.record()
        torch.cuda.synchronize()
        out[label] = round(4.0 * n / (e0.elapsed_time(e1) / 10 * 1e-3) / 1e9, 1)
        del x
    return out


def ceiling(dev):
    """`--ceiling`: what the engines under a bf16 GEMM's K loop deliver on this GPU in this run, from probe kernels of
    the library (dion_amd_probe): matrix cores alone (random operands in registers) with the shader clock they ran at,
    and the L2 -> LDS stream of the operand staging alone."""
    import ctypes

    import torch
    from dion_amd import _lib

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    src = torch.randn(max(cus * 49152, (cus + 31) // 32 * 65536) // 2, device=dev).bfloat16()
    rec = torch.zeros(cus * 8 * 4, dtype=torch.int64, device=dev)
    sink = torch.zeros(1, device=dev)
    out = {}
    for which, name, iters in ((0, "mfma_only", 20000), (4, "mfma_only_16x16x32", 20000), (1, "l2_to_lds_stream", 20000),
                               (2, "l2_to_vgpr_stream", 20000), (3, "lds_read_stream", 20000)):
        best = None
        for _ in range(3):
            ms = ctypes.c_double(0)
            _lib.check(lib.dion_amd_probe(which, src.data_ptr(), src.numel() * 2, iters, rec.data_ptr(), rec.numel() * 8,
                                          sink.data_ptr(), ctypes.byref(ms), _lib.stream_ptr(dev)), "dion_amd_probe")
            r = rec.cpu().view(-1, 4)
            mhz = float((r[:, 3] - r[:, 2]).sum()) / float((r[:, 1] - r[:, 0]).sum()) * 100.0
            if best is None or ms.value < best[0]:
                best = (ms.value, mhz)
        ms, mhz = best
        if which in (0, 4):
            flops = cus * 8 * iters * (32 * 32768.0 if which == 0 else 64 * 16384.0)
            out[name] = dict(pflops=round(flops / (ms * 1e-3) / 1e15, 3), frac_of_2_5_pflops=round(flops / (ms * 1e-3) / PEAK_BF16_FLOPS, 3),
                             shader_clock_mhz=round(mhz), ms=round(ms, 3),
                             peak_at_that_clock_pflops=round(cus * 4096 * mhz * 1e6 / 1e15, 3))
        else:
            nbytes = cus * iters * 65536.0
            out[name] = dict(tbps=round(nbytes / (ms * 1e-3) / 1e12, 2), shader_clock_mhz=round(mhz), ms=round(ms, 3),
                             bytes_per_clock_per_cu=round(nbytes / cus / (ms * 1e-3) / (mhz * 1e6), 1))
    out["streaming_kernel_gbps"] = stream_ceiling(dev)
    return out


def vendor_matmul(dev):
    """`--vendor-matmul`: the three Newton-Schulz products of 4096 x 14336 matrices (a bucket of 32) as plain out-of-place
    `torch.matmul` calls (the vendor GEMM library) next to this library's kernels on the same operands in the same run.
    Dense flops 2 M N K for both, so the symmetric kernels' figures count the half they do not execute."""
    import torch
    from dion_amd.newton_schulz import gemm, ns_line_1, ns_line_2

    bf = torch.bfloat16
    b, m, n = 32, 4096, 14336
    X = (torch.randn(b, m, n, device=dev) * 0.01).to(bf)
    A = (torch.randn(b, m, m, device=dev) * 0.01).to(bf)
    A = ((A + A.mT) * 0.5).contiguous()
    Y = torch.empty_like(X)
    A2 = torch.empty_like(A)

    def timed(fn, reps=5):
        for _ in range(2):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    cases = {
        "X X^T (32 x 4096x14336)": (2.0 * b * m * m * n, lambda: torch.matmul(X, X.mT, out=A2), lambda: ns_line_1(X, out=A2)),
        "A A (32 x 4096^3)": (2.0 * b * m * m * m, lambda: torch.matmul(A, A, out=A2),
                             lambda: ns_line_2(A, 2.0315, -4.775, out=A2, faithful=True)),
        "B X (32 x 4096x4096x14336)": (2.0 * b * m * m * n, lambda: torch.matmul(A, X, out=Y),
                                      lambda: gemm(A, X, b_kstrided=True, E=X, s0=3.4445, s1=1.0, out=Y, faithful=True)),
    }
    out = {}
    for name, (flops, vend, ours) in cases.items():
        tv, to = timed(vend), timed(ours)
        out[name] = dict(vendor_ms=round(tv, 3), vendor_dense_pflops=round(flops / (tv * 1e-3) / 1e15, 3),
                         this_library_ms=round(to, 3), this_library_dense_pflops=round(flops / (to * 1e-3) / 1e15, 3),
                         note="this library's launch includes the rounding-faithful epilogue (and the polynomial / axpy "
                              "combine) and runs here on contiguous operands (row pitch a multiple of 4 KiB; the "
                              "optimizer's working matrices carry 128 bytes of padding: see workload muon_4096x14336)")
    return out


def tile_trace(dev):
    """Time line of single bf16 GEMM launches (`--tile-trace`): per output tile, when its workgroup started, finished
    its K loop and finished its epilogue, and on which CU.  Prints one summary line per product: mean duration of the
    two phases, the gap until the CU's next workgroup, and how many tiles were in their epilogue at 40 instants of the
    launch (all-or-nothing values mean that the CUs run in lockstep)."""
    import ctypes

    import numpy as np
    import torch
    from dion_amd import _lib
    from dion_amd.newton_schulz import gemm

    lib = _lib.load()
    torch.manual_seed(0)

    def report(name, ntiles):
        ntiles = min(ntiles, 65536)
        buf = np.zeros((ntiles, 6), dtype=np.uint64)
        _lib.check(lib.dion_amd_tile_trace_read(ctypes.c_void_p(buf.ctypes.data), ntiles), "dion_amd_tile_trace_read")
        t0, t1, t2 = (buf[:, i].astype(np.int64) for i in range(3))
        hw = buf[:, 3]
        xcc = (hw >> np.uint64(32)).astype(np.int64)
        h = (hw & np.uint64(0xffffffff)).astype(np.int64)
        cu = ((xcc * 8 + ((h >> 13) & 7)) * 2 + ((h >> 12) & 1)) * 16 + ((h >> 8) & 15)
        gaps = []
        for c in np.unique(cu):
            idx = np.where(cu == c)[0]
            o = idx[np.argsort(t0[idx])]
            gaps += ((t0[o][1:] - t2[o][:-1]) / 100.0).tolist()
        mhz = (buf[:, 5].astype(np.int64) - buf[:, 4].astype(np.int64)) / np.maximum(t2 - t0, 1) * 100.0
        ts = np.linspace(t0.min(), t2.max(), 40)
        in_epi = [int(((t1 <= x) & (t2 > x)).sum()) for x in ts]
        print(json.dumps(dict(
            product=name, tiles=int(ntiles), cus=int(len(np.unique(cu))), launch_us=round((t2.max() - t0.min()) / 100.0, 1),
            k_loop_us=round(float(((t1 - t0) / 100.0).mean()), 2), epilogue_us=round(float(((t2 - t1) / 100.0).mean()), 2),
            gap_us=round(float(np.mean(gaps)), 2) if gaps else None,
            shader_clock_mhz=dict(mean=round(float(mhz.mean())), p10=round(float(np.percentile(mhz, 10))),
                                  p90=round(float(np.percentile(mhz, 90)))),
            tiles_in_epilogue_at_40_instants=in_epi)))

    def run(name, fn, ntiles):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        lib.dion_amd_tile_trace_enable(1)
        fn()
        lib.dion_amd_tile_trace_enable(0)
        report(name, ntiles)

    bf = torch.bfloat16
    # Dion error feedback M <- M - 0.05 P R^T, in place, 4 x (28672 x 8192), rank 512 and rank 64
    for r in (512, 64):
        P = (torch.randn(4, 28672, r, device=dev) * 0.03).to(bf)
        R = (torch.randn(4, 8192, r, device=dev) * 0.03).to(bf)
        M = torch.randn(4, 28672, 8192, device=dev).to(bf)
        run(f"M + a P R^T, 4 x 28672x8192, rank {r}", lambda: gemm(P, R, E=M, s0=1.0, s1=-0.05, out=M, faithful=True),
            4 * 112 * 32)
        del P, R, M
    # Newton-Schulz X' = aX + BX: 24 x (768 x 3072) and 4 x (4096 x 4096)
    for b, m, n in ((24, 768, 3072), (4, 4096, 4096)):
        X = (torch.randn(b, m, n, device=dev) * 0.03).to(bf)
        B = (torch.randn(b, m, m, device=dev) * 0.03).to(bf)
        Y = torch.empty_like(X)
        run(f"X' = aX + BX, {b} x {m}x{n}", lambda: gemm(B, X, b_kstrided=True, E=X, s0=3.0, s1=1.0, out=Y, faithful=True),
            b * (m // 256) * (n // 256))
        del X, B, Y
    # A = X X^T (upper tiles) on b x (768 x 3072): 6 b tiles of 48 stages each, one per CU while 6 b <= 256 -- the
    # same tile program on 48 ... 252 busy CUs
    from dion_amd.newton_schulz import ns_line_1
    for b in (8, 24, 32, 40, 42):
        X = (torch.randn(b, 768, 3072, device=dev) * 0.03).to(bf)
        A = torch.empty(b, 768, 768, device=dev, dtype=bf)
        run(f"A = X X^T, {b} x 768x3072 ({6 * b} tiles)", lambda: ns_line_1(X, out=A), 6 * b)
        del X, A


def flow_trace(dev):
    """`--flow-trace`: time line of the persistent Newton-Schulz launch of one GPT-small Muon step.  Per tile the kernel
    records when its workgroup took it up, when its dependency was met, when its K loop and when its epilogue ended.
    One JSON line: per product the mean of the three phases, and per compute unit the sums."""
    import ctypes

    import numpy as np
    import torch
    from dion_amd import _lib

    lib = _lib.load()
    opt, params, _ = build_optimizer(WORKLOADS["muon_gpt_small"], dev)
    for _ in range(5):
        opt.step()
    torch.cuda.synchronize()
    lib.dion_amd_ns_flow_trace_enable(1)
    opt.step()
    torch.cuda.synchronize()
    lib.dion_amd_ns_flow_trace_enable(0)
    cap = 65536
    buf = np.zeros((cap, 6), dtype=np.uint64)
    n = ctypes.c_int(0)
    _lib.check(lib.dion_amd_ns_flow_trace_read(ctypes.c_void_p(buf.ctypes.data), cap, ctypes.byref(n)),
               "dion_amd_ns_flow_trace_read")
    buf = buf[:n.value]
    t = (buf[:, :4].astype(np.int64) - buf[:, 0].astype(np.int64).min()) / 100.0   # microseconds
    phase = ((buf[:, 4] >> np.uint64(32)) & np.uint64(0xffff)).astype(int)
    wait, kloop, epi = t[:, 1] - t[:, 0], t[:, 2] - t[:, 1], t[:, 3] - t[:, 2]
    cus = len(np.unique(buf[:, 5]))
    # gaps between consecutive tiles of a compute unit
    order = np.argsort(t[:, 0])
    last, gaps = {}, []
    for i in order:
        k = int(buf[i, 5])
        if k in last:
            gaps.append(t[i, 0] - last[k])
        last[k] = t[i, 3]
    out = dict(tiles=int(n.value), compute_units=int(cus), launch_us=round(float(t[:, 3].max()), 1), products={})
    for p, name in enumerate(("A = X X^T", "B = bA + cAA", "X' = aX + BX")):
        m = (phase % 3) == p
        out["products"][name] = dict(tiles=int(m.sum()), wait_us=round(float(wait[m].mean()), 2),
                                     k_loop_us=round(float(kloop[m].mean()), 2),
                                     epilogue_us=round(float(epi[m].mean()), 2))
    out["per_compute_unit_us"] = dict(wait=round(float(wait.sum() / cus), 1), k_loop=round(float(kloop.sum() / cus), 1),
                                      epilogue=round(float(epi.sum() / cus), 1),
                                      between_tiles=round(float(np.sum(gaps) / cus), 1))
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="muon_gpt_small", choices=sorted(WORKLOADS))
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--tile-trace", action="store_true",
                    help="instead of a workload: time lines of single bf16 GEMM launches (one JSON line per product)")
    ap.add_argument("--flow-trace", action="store_true",
                    help="instead of a workload: per-tile time line of the persistent Newton-Schulz launch (GPT-small)")
    ap.add_argument("--ceiling", action="store_true",
                    help="instead of a workload: matrix-core-only and L2->LDS-only probe kernels with the shader clock")
    ap.add_argument("--vendor-matmul", action="store_true",
                    help="instead of a workload: torch.matmul on the 4096x14336 Newton-Schulz products next to this library")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run three plain 512 MiB device copies (reference point for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    if args.flow_trace:
        flow_trace(dev)
        return
    if args.tile_trace:
        tile_trace(dev)
        return
    if args.ceiling:
        print(json.dumps(dict(device=device_info(dev), ceiling=ceiling(dev))))
        return
    if args.vendor_matmul:
        print(json.dumps(dict(device=device_info(dev), products=vendor_matmul(dev))))
        return
    if args.calibrate_copy:
        src = torch.ones(512 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    wl = WORKLOADS[args.workload]
    res = measure(wl, dev, args.steps, args.warmup)
    main_sum = summarize(args.workload, wl, res)

    out = {
        "metric": "Muon/Dion optimizer-step ms (GPT-160M, 8B-layer) + % bf16 MFMA peak",
        "value": round(res["ms_per_step"], 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": args.workload, "description": wl["desc"], "matrices": len(wl["shapes"]),
                   "optimizer": res["optimizer"], "grad": f"N(0,1e-3) seed {wl['seed']}", "parallelism": "single GPU"},
        "event_ms_per_step": round(res["event_ms"], 4),
        "wall_ms_per_step": round(res["wall_ms"], 4),
        "roofline": roofline_of(res, wl["kind"], args.workload, dion_hbm_bytes(wl) if wl["kind"] == "dion" else None),
        "device": device_info(dev),
    }
    out["device"]["streaming_kernel_gbps"] = stream_ceiling(dev)
    out.update({k: v for k, v in main_sum.items() if k not in ("workload", "ms_per_step", "steps")})
    if not args.no_extra:
        extra = {}
        for name in ("dion_gpt_small_r025", "dion_gpt_small_r1", "muon_llama8b_layer", "muon_4096x14336", "dion_llama70b_layer",
                     "muon_llama8b", "dion_llama70b_mlp", "scalar_gpt_small"):
            if name == args.workload:
                continue
            w = WORKLOADS[name]
            big = name in ("muon_llama8b", "dion_llama70b_mlp", "muon_4096x14336")   # hundreds of ms and tens of GB per step
            r = measure(w, dev, 3 if big else 10, 1 if big else 2)
            s = summarize(name, w, r)
            s["roofline"] = roofline_of(r, w["kind"], name, dion_hbm_bytes(w) if w["kind"] == "dion" else None)
            extra[name] = s
        out["extra"] = extra
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
