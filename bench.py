#!/usr/bin/env python3
"""Benchmark of the Muon optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b|gpt2-124m|ns32|conv]

A step is one full SingleDeviceMuonWithAuxAdam.step() over the synthetic parameter set of the
workload (seeded random parameters and gradients resident in HBM before the timed region starts;
the K timed steps run back to back between two device synchronisations).  Prints
one JSON line: step time, the MFMA roofline of the Newton-Schulz GEMM launches measured with HIP
events on the launch stream, the HBM fractions of the elementwise kernels, and the CPU baseline
(the oracle restatement of the reference timed on the host cores over a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
# HBM-side bytes per ns_gemm launch (FETCH_SIZE + WRITE_SIZE of two rocprofv3 --pmc runs of this
# script, scaled by what the counters read for a 1 GiB copy; averaged over the launches of a step)
GEMM_TRAFFIC_BYTES_PER_LAUNCH = {"llama3-8b": 1.950e10}


# ------------------------------------------------------------------------------------------
# workloads: the benchmark configurations (parameter sets of GPT-2-small, Llama-3-8B, a CIFAR ConvNet)
# ------------------------------------------------------------------------------------------
def workload_shapes(name):
    """-> (muon [(shape, count)], adam [(shape, count)], grad_std, default_steps, default_warmup)"""
    if name == "llama3-8b":
        muon = [((4096, 4096), 64), ((1024, 4096), 64), ((14336, 4096), 64), ((4096, 14336), 32)]
        adam = [((128256, 4096), 2), ((4096,), 65)]
        return muon, adam, 1e-4, 3, 1
    if name == "gpt2-124m":
        muon = [((768, 2304), 12), ((768, 768), 12), ((768, 3072), 12), ((3072, 768), 12)]
        adam = [((50257, 768), 1), ((1024, 768), 1), ((768,), 25)]
        return muon, adam, 1e-3, 10, 3
    if name == "conv":
        muon = [((64, 24, 3, 3), 1), ((256, 64, 3, 3), 1), ((256, 256, 3, 3), 2), ((512, 256, 3, 3), 1),
                ((512, 512, 3, 3), 3), ((128, 16384), 1), ((16384, 128), 1)]
        adam = [((24, 3, 2, 2), 1), ((10, 512), 1)]
        return muon, adam, 1e-2, 10, 3
    raise ValueError(name)


def f_sym(m, n, steps=5):
    return steps * (m * (m + 1) * n + m * m * (m + 1) + 2 * m * m * n)


def f_dense(m, n, steps=5):
    return steps * (4 * m * m * n + 2 * m ** 3)


def mat2d(shape):
    rows = shape[0]
    cols = 1
    for s in shape[1:]:
        cols *= s
    return rows, cols


# ------------------------------------------------------------------------------------------
# GPU leg
# ------------------------------------------------------------------------------------------
def run_optimizer_workload(name, steps, warmup, seed, ns_variant="ns5", use_graph=False):
    import muon_amd
    from muon_amd import engine

    muon, adam, gstd, _, _ = workload_shapes(name)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    pm, pa = [], []
    for shape, count in muon:
        for _ in range(count):
            pm.append(torch.nn.Parameter(torch.randn(*shape, device=dev, generator=gen) * 0.02))
    for shape, count in adam:
        for _ in range(count):
            init = torch.ones(*shape, device=dev) if len(shape) == 1 else torch.randn(*shape, device=dev, generator=gen) * 0.02
            pa.append(torch.nn.Parameter(init))
    for p in pm + pa:
        p.grad = torch.empty_like(p)
    opt = muon_amd.SingleDeviceMuonWithAuxAdam([
        dict(params=pm, use_muon=True, lr=0.02, momentum=0.95, weight_decay=0.01),
        dict(params=pa, use_muon=False, lr=3e-4, betas=(0.9, 0.95), eps=1e-10, weight_decay=0.01)],
        ns_variant=ns_variant, use_graph=use_graph)

    # The gradients stay resident and unchanged over the run (the step does not write them); the
    # momentum and the parameters move every step, so every step orthogonalises new matrices.
    for p in pm + pa:
        p.grad.normal_(0.0, gstd, generator=gen)
    for _ in range(warmup):
        opt.step()
    torch.cuda.synchronize()

    # timed region: exactly `steps` steps back to back, one synchronisation on either side; a pair
    # of HIP events on the launch stream brackets every kernel launch inside it
    engine.PROFILE = None if use_graph else []      # a replayed graph has no per-launch events
    t0 = time.perf_counter()
    for _ in range(steps):
        opt.step()
    torch.cuda.synchronize()
    total_ms = (time.perf_counter() - t0) * 1e3
    prof, engine.PROFILE = engine.PROFILE or [], None

    per_label = {}
    for label, work, e0, e1 in prof:
        d = per_label.setdefault(label, [0.0, 0.0, 0])
        d[0] += work
        d[1] += e0.elapsed_time(e1)
        d[2] += 1
    n_m = sum(p.numel() for p in pm)
    n_a = sum(p.numel() for p in pa)
    fs = sum(f_sym(min(mat2d(s)), max(mat2d(s))) * c for s, c in muon)
    fd = sum(f_dense(min(mat2d(s)), max(mat2d(s))) * c for s, c in muon)
    # sanity: the state after the timed steps is finite
    assert all(torch.isfinite(p).all() for p in pm[:2] + pa[:2])
    del opt, pm, pa
    torch.cuda.empty_cache()
    return dict(ms_per_step=total_ms / steps, per_label=per_label, muon_elements=n_m, adam_elements=n_a,
                f_sym=fs, f_dense=fd)


def summarize_kernels(per_label):
    out = {}
    gemm_work = gemm_ms = gemm_n = 0
    for label, (work, ms, n) in sorted(per_label.items()):
        if label.startswith("ns_gemm"):
            gemm_work += work
            gemm_ms += ms
            gemm_n += n
            out[label] = dict(launches=n, avg_ms=ms / n, tflops=work / ms / 1e9, frac_of_peak=work / ms / 1e9 / PEAK_BF16_TFLOPS)
        else:
            out[label] = dict(launches=n, avg_ms=ms / n, gbs=work / ms / 1e6, frac_of_peak=work / ms / 1e6 / PEAK_HBM_GBS)
    return out, gemm_work, gemm_ms, gemm_n


def run_ns32(steps, warmup, seed):
    """Benchmark configuration 3: 32 independent 4096 x 4096 bf16 matrices ~N(0,1) through
    zeropower_via_newtonschulz5 (5 iterations); one call is one step."""
    import muon_amd
    from muon_amd import engine

    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(seed)
    G = torch.randn(32, 4096, 4096, device="cuda:0", generator=gen).bfloat16()
    for _ in range(warmup):
        muon_amd.zeropower_via_newtonschulz5(G)
    torch.cuda.synchronize()
    engine.PROFILE = []
    t0 = time.perf_counter()
    for _ in range(steps):
        out = muon_amd.zeropower_via_newtonschulz5(G)
    torch.cuda.synchronize()
    total_ms = (time.perf_counter() - t0) * 1e3
    prof, engine.PROFILE = engine.PROFILE, None
    assert torch.isfinite(out[0]).all()
    per_label = {}
    for label, work, e0, e1 in prof:
        d = per_label.setdefault(label, [0.0, 0.0, 0])
        d[0] += work
        d[1] += e0.elapsed_time(e1)
        d[2] += 1
    muon_amd.clear_engine_cache()
    return dict(ms_per_step=total_ms / steps, per_label=per_label, muon_elements=32 * 4096 * 4096, adam_elements=0,
                f_sym=32 * f_sym(4096, 4096), f_dense=32 * f_dense(4096, 4096))


# ------------------------------------------------------------------------------------------
# CPU baseline: the oracle restatement of the reference on the host cores, bounded sample
# ------------------------------------------------------------------------------------------
def cpu_baseline(name, budget_s=25.0):
    from oracle import muon_oracle as O
    cores = min(16, os.cpu_count() or 1)
    torch.set_num_threads(cores)
    muon, adam, gstd, _, _ = workload_shapes(name)
    torch.manual_seed(4321)
    total_ms, parts, t_start = 0.0, [], time.perf_counter()
    # one instance of each distinct Muon shape; a shape and its transpose cost the same (the
    # iteration runs on the wide orientation either way), so they share one timing
    merged = {}
    for shape, count in muon:
        r, c = mat2d(shape)
        key = (min(r, c), max(r, c))
        merged[key] = (shape if key not in merged else merged[key][0], count + (merged[key][1] if key in merged else 0))
    for _, (shape, count) in sorted(merged.items(), key=lambda kv: kv[0][0] * kv[0][1]):
        if time.perf_counter() - t_start > budget_s:
            parts.append(f"{shape}: skipped (budget)")
            continue
        p = torch.nn.Parameter(torch.randn(*shape) * 0.02)
        p.grad = torch.randn(*shape) * gstd
        opt = O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p], use_muon=True, lr=0.02, weight_decay=0.01)])
        t0 = time.perf_counter()
        opt.step()
        ms = (time.perf_counter() - t0) * 1e3
        total_ms += ms * count
        parts.append(f"{count}x{tuple(shape)}@{ms:.0f}ms")
    # Adam: one slab of at most 4096 rows of each distinct shape, scaled by element count
    for shape, count in adam:
        rows = min(shape[0], 4096)
        sl = (rows,) + tuple(shape[1:])
        p = torch.nn.Parameter(torch.randn(*sl) * 0.02)
        p.grad = torch.randn(*sl) * gstd
        opt = O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p], use_muon=False, weight_decay=0.01)])
        t0 = time.perf_counter()
        opt.step()
        ms = (time.perf_counter() - t0) * 1e3 * (shape[0] / rows)
        total_ms += ms * count
    skipped = any("skipped" in s for s in parts)
    return dict(value=None if skipped else round(total_ms, 1), unit="ms/step", cores=cores, kind="port",
                sample="one oracle step per distinct Muon shape and one <=4096-row slab per Adam shape, "
                       "summed as count x time (extrapolated): " + ", ".join(parts))


# ------------------------------------------------------------------------------------------
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="llama3-8b", choices=["llama3-8b", "gpt2-124m", "conv", "ns32"])
    ap.add_argument("--ns-variant", default="ns5", choices=["ns5", "aol4"],
                    help="ns5: the five-iteration specification (the headline); aol4: the 4-iteration "
                         "AOL-rescaled variant (its flop count is 11/15 of the headline's, so only the step "
                         "time of such a run is comparable, not the roofline fraction)")
    ap.add_argument("--graph", action="store_true",
                    help="replay the Muon launches from a HIP graph (use_graph=True): step time only, the "
                         "per-kernel figures need the eager launches")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary GPT-2 measurement")
    ap.add_argument("--copy-probe", action="store_true",
                    help="first run one plain 1 GiB device-to-device copy kernel (a known-size reference "
                         "for scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the Muon update shards "
                 "by matrix across ranks, which is not part of this library). Run with --gpus 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X GPU")
    if args.workload == "ns32":
        steps = args.steps if args.steps is not None else 5
        warmup = args.warmup if args.warmup is not None else 1
        res = run_ns32(steps, warmup, seed=1234 + 3)
        kernels, gemm_work, gemm_ms, gemm_n = summarize_kernels(res["per_label"])
        print(json.dumps({
            "metric": "ns5_ms_32x4096x4096_bf16", "value": round(res["ms_per_step"], 3), "unit": "ms", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": round(res["ms_per_step"], 3),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "ns32: zeropower_via_newtonschulz5 on 32 x 4096 x 4096 bf16 ~N(0,1), 5 iterations",
                       "rounding": "reference"},
            "roofline": {"bound": "mfma", "kernel": "ns_gemm_kernel (syrk + poly + update launches)",
                         "achieved": round(gemm_work / gemm_ms / 1e9, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(gemm_work / gemm_ms / 1e9 / PEAK_BF16_TFLOPS, 4), "traffic": None,
                         "launches": gemm_n, "avg_launch_ms": round(gemm_ms / gemm_n, 4),
                         "flops_per_launch": gemm_work / gemm_n},
            "ns": {"tflops_sym_whole_call": round(res["f_sym"] / res["ms_per_step"] / 1e9, 1),
                   "tflops_dense_equiv_whole_call": round(res["f_dense"] / res["ms_per_step"] / 1e9, 1)},
            "kernels": {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in kernels.items()},
        }))
        return
    _, _, _, dsteps, dwarm = workload_shapes(args.workload)
    steps = args.steps if args.steps is not None else dsteps
    warmup = args.warmup if args.warmup is not None else dwarm

    if args.copy_probe:
        a = torch.ones(1 << 28, dtype=torch.float32, device="cuda:0")      # 1 GiB
        b = torch.empty_like(a)
        b.copy_(a)                                                            # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del a, b
    res = run_optimizer_workload(args.workload, steps, warmup, seed=1234 + 4, ns_variant=args.ns_variant,
                                 use_graph=args.graph)
    if args.graph:
        print(json.dumps({"metric": f"muon_step_ms_{args.workload}", "value": round(res["ms_per_step"], 3),
                          "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warmup,
                          "ms_per_step": round(res["ms_per_step"], 3), "higher_is_better": False,
                          "config": {"workload": args.workload, "ns_variant": args.ns_variant, "launch": "hip graph replay"}}))
        return
    kernels, gemm_work, gemm_ms, gemm_n = summarize_kernels(res["per_label"])
    ew_bytes = sum(w for l, (w, ms, n) in res["per_label"].items() if not l.startswith("ns_gemm"))
    ew_ms = sum(ms for l, (w, ms, n) in res["per_label"].items() if not l.startswith("ns_gemm"))
    line = {
        "metric": f"muon_step_ms_{args.workload}",
        "value": round(res["ms_per_step"], 3),
        "unit": "ms",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(res["ms_per_step"], 3),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: full SingleDeviceMuonWithAuxAdam step, fp32 params/grads/state, "
                               f"{res['muon_elements']} Muon + {res['adam_elements']} Adam elements, "
                               "lr .02 wd .01 momentum .95 nesterov ns_steps 5; Adam lr 3e-4 betas (.9,.95)",
                   "rounding": "reference" if args.ns_variant == "ns5" else "one rounding per stored matrix",
                   "ns_variant": args.ns_variant},
        "roofline": {
            "bound": "mfma",
            "kernel": "ns_gemm_kernel (syrk + poly + update launches)",
            "achieved": round(gemm_work / gemm_ms / 1e9, 1),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gemm_work / gemm_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
            "traffic": GEMM_TRAFFIC_BYTES_PER_LAUNCH.get(args.workload),
            "launches": gemm_n,
            "avg_launch_ms": round(gemm_ms / gemm_n, 4),
            "flops_per_launch": gemm_work / gemm_n,
        },
        "ns": {
            "ns_ms_per_step": round(gemm_ms / steps, 3),
            "tflops_sym": round(res["f_sym"] * steps / gemm_ms / 1e9, 1),
            "tflops_dense_equiv": round(res["f_dense"] * steps / gemm_ms / 1e9, 1),
        },
        "elementwise": {
            "ms_per_step": round(ew_ms / steps, 3),
            "launched_gbs": round(ew_bytes / ew_ms / 1e6, 1),
            "algorithmic_gbs": round((res["muon_elements"] * 24 + res["adam_elements"] * 28) * steps / ew_ms / 1e6, 1),
            "frac_of_hbm_peak_algorithmic": round((res["muon_elements"] * 24 + res["adam_elements"] * 28) * steps / ew_ms / 1e6 / PEAK_HBM_GBS, 4),
        },
        "kernels": {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in kernels.items()},
    }
    if not args.no_extra and args.workload == "llama3-8b":
        g = run_optimizer_workload("gpt2-124m", 10, 3, seed=1234 + 2)
        _, gw, gms, _ = summarize_kernels(g["per_label"])
        gg = run_optimizer_workload("gpt2-124m", 10, 3, seed=1234 + 2, use_graph=True)
        line["gpt2_124m"] = {"ms_per_step": round(g["ms_per_step"], 3), "ns_tflops_sym": round(gw / gms / 1e9, 1),
                             "ms_per_step_graph_replay": round(gg["ms_per_step"], 3)}
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.workload)
        if line["cpu_baseline"]["value"]:
            line["cpu_baseline"]["gpu_speedup"] = round(line["cpu_baseline"]["value"] / res["ms_per_step"], 1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
