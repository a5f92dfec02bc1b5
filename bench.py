#!/usr/bin/env python3
"""Benchmark of the Muon optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b|gpt2-124m|ns32|conv]

A step is one full SingleDeviceMuonWithAuxAdam.step() over the synthetic parameter set of the
workload (seeded random parameters and gradients resident in HBM before the timed region starts;
the K timed steps run back to back between two device synchronisations).  Before anything is timed
the HIP path is checked against the CPU oracle on the shapes of the workload (Newton-Schulz within
2e-2 of the bf16 restatement and 3e-2 of fp32, parameters within 1e-3 after a step, Adam within
1e-5); a failed gate ends the run with a non-zero exit code and no JSON line.  Prints one JSON
line: step time, the MFMA roofline of the Newton-Schulz GEMM launches measured with HIP events on
the launch stream, the HBM fractions of the elementwise kernels, the other benchmark configurations
as sub-objects, and the CPU baseline (the oracle restatement of the reference timed on the host
cores over a bounded sample).
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
# HBM-side bytes per ns_gemm launch: NOT measured by this script.  The figure comes from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE, scaled by what the counters read for
# a 1 GiB copy, averaged over the launches of a step); the summary file is named beside it.
GEMM_TRAFFIC_BYTES_PER_LAUNCH = {"llama3-8b": (3.02e10, "profiles/hbm_traffic_llama3-8b_step.md")}

TOL_NS_BF16, TOL_NS_FP32, TOL_PARAM, TOL_ADAM = 2e-2, 3e-2, 1e-3, 1e-5


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


def workload_bounds(name):
    """Lower bounds of one optimizer step of a workload on an MI355X.
    mfma_ms: the symmetric-minimum Newton-Schulz flops at the dense bf16 peak.
    hbm_elementwise_ms: 24 B per Muon element + 28 B per Adam element at the HBM peak.
    hbm_ns_ms: the Newton-Schulz intermediates through HBM once per product, 5 * (6 m n + 8 m^2) bytes
    per matrix (X read twice and written once, A and B written and read once, bf16): what bounds the
    iteration of matrices too short (m < ~640) for their products to be MFMA-bound."""
    muon, adam, _, _, _ = workload_shapes(name)
    fs = ns_bytes = n_m = n_a = 0
    for shape, count in muon:
        r, c = mat2d(shape)
        m, n = min(r, c), max(r, c)
        fs += count * f_sym(m, n)
        ns_bytes += count * 5 * (6 * m * n + 8 * m * m)
        n_m += count * r * c
    for shape, count in adam:
        r, c = mat2d(shape)
        n_a += count * r * c
    ew_bytes = 24 * n_m + 28 * n_a
    return dict(mfma_ms=fs / (PEAK_BF16_TFLOPS * 1e9), hbm_elementwise_ms=ew_bytes / (PEAK_HBM_GBS * 1e6),
                hbm_ns_ms=ns_bytes / (PEAK_HBM_GBS * 1e6), ns_bytes=ns_bytes, elementwise_bytes=ew_bytes)


def mat2d(shape):
    rows = shape[0]
    cols = 1
    for s in shape[1:]:
        cols *= s
    return rows, cols


# ------------------------------------------------------------------------------------------
# correctness gates (run before anything is timed)
# ------------------------------------------------------------------------------------------
def correctness_gates(name):
    """The HIP path against the CPU oracle on one instance of every distinct Muon shape of the
    workload (Newton-Schulz output and one optimizer step) and on a slab of every Adam shape.
    Returns the measured distances; ends the run when one exceeds its bound."""
    import muon_amd
    from oracle import muon_oracle as O

    torch.set_num_threads(host_threads())
    res, failed = {}, []
    res["effective_bounds"], res["parity_unpinned"] = {}, []

    def gate(key, value, bound, nominal=None):
        """`nominal`: the bound the contract states, when `bound` is a widened one.  A gate that
        passes only through the widening is listed under "parity_unpinned" instead of counting as
        a plain pass."""
        res[key] = round(float(value), 6)
        res["effective_bounds"][key] = round(float(bound), 6)
        if not value <= bound:
            failed.append(f"{key} = {value:.3e} > {bound:.3e}")
        elif nominal is not None and not value <= nominal:
            res["parity_unpinned"].append(f"{key}: {float(value):.3e} is above the stated {nominal:.0e}, "
                                          f"within the widened {float(bound):.3e}")

    def ns_gates(tag, g2):
        """Newton-Schulz output for the 2-D input g2 (CPU tensor).  The oracle's bf16 tensor
        expressions are evaluated twice: by torch on the CPU, and by torch on this GPU (bf16
        torch.matmul = rocBLAS, the library the reference itself multiplies with).  Both accumulate
        in fp32 but in different orders, and on strongly rectangular matrices (4096 x 14336) the
        iteration amplifies that to more than 2e-2 between the two evaluations of the SAME
        expressions; the bound on the distance to the CPU evaluation is therefore the larger of 2e-2
        and the distance between the two evaluations (+5e-3).  The distance to the GPU evaluation
        is held to 2e-2 everywhere."""
        got = muon_amd.zeropower_via_newtonschulz5(g2.cuda()).float().cpu()
        ref16, ref32 = O.ns5_bf16(g2).float(), O.ns5_fp32(g2.float())
        ref16_gpu = O.ns5_bf16(g2.cuda()).float().cpu()
        spread = O.rel_fro(ref16_gpu, ref16)
        res[f"ns_bf16_oracle_cpu_vs_gpu_evaluation_{tag}"] = round(float(spread), 6)
        gate(f"ns_vs_bf16_gpu_evaluated_{tag}", O.rel_fro(got, ref16_gpu), TOL_NS_BF16)
        gate(f"ns_vs_bf16_{tag}", O.rel_fro(got, ref16), max(TOL_NS_BF16, spread + 5e-3), TOL_NS_BF16)
        # where the reference's own bf16 result is further than 3e-2 from fp32 (small conv
        # shapes), the kernel that follows its rounding sequence inherits that distance
        gate(f"ns_vs_fp32_{tag}", O.rel_fro(got, ref32), max(TOL_NS_FP32, O.rel_fro(ref16, ref32) + 5e-3), TOL_NS_FP32)

    torch.manual_seed(97)
    if name == "ns32":
        ns_gates("4096x4096", torch.randn(4096, 4096).bfloat16())
    else:
        muon, adam, gstd, _, _ = workload_shapes(name)
        for shape, _ in muon:
            tag = "x".join(str(v) for v in shape)
            p_c = torch.nn.Parameter(torch.randn(*shape) * 0.02)
            p_g = torch.nn.Parameter(p_c.detach().clone().cuda())
            g = torch.randn(*shape) * gstd
            p_c.grad, p_g.grad = g.clone(), g.clone().cuda()
            ns_gates(tag, g.reshape(mat2d(shape)))
            O.OracleSingleDeviceMuon([p_c], lr=0.02, weight_decay=0.01, momentum=0.95).step()
            muon_amd.SingleDeviceMuon([p_g], lr=0.02, weight_decay=0.01, momentum=0.95).step()
            # a tiny filter's update is several per cent of |p|, so bf16 Newton-Schulz noise weighs more there
            gate(f"param_after_step_{tag}", O.rel_fro(p_g.detach().cpu(), p_c.detach()),
                 TOL_PARAM if min(mat2d(shape)) >= 128 else 3e-3, TOL_PARAM)
        for shape, _ in adam:
            sl = (min(shape[0], 4096),) + tuple(shape[1:])
            tag = "x".join(str(v) for v in sl)
            p_c = torch.nn.Parameter(torch.randn(*sl) * 0.02)
            p_g = torch.nn.Parameter(p_c.detach().clone().cuda())
            kw = dict(use_muon=False, lr=3e-4, betas=(0.9, 0.95), eps=1e-10, weight_decay=0.01)
            oc = O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p_c], **kw)])
            og = muon_amd.SingleDeviceMuonWithAuxAdam([dict(params=[p_g], **kw)])
            for _ in range(2):
                g = torch.randn(*sl) * gstd
                p_c.grad, p_g.grad = g.clone(), g.clone().cuda()
                oc.step()
                og.step()
            d = (p_g.detach().cpu() - p_c.detach()).abs() / p_c.detach().abs().clamp_min(1e-3)
            gate(f"adam_max_rel_{tag}", d.max(), TOL_ADAM)
    muon_amd.clear_engine_cache()
    torch.cuda.empty_cache()
    if failed:
        sys.exit("bench.py: correctness gate failed before timing: " + "; ".join(failed))
    return res


# ------------------------------------------------------------------------------------------
# GPU leg
# ------------------------------------------------------------------------------------------
def run_optimizer_workload(name, steps, warmup, seed, ns_variant="ns5", use_graph=False, realloc_grads=False,
                           launch_events=True):
    import muon_amd
    from muon_amd import engine, plan

    # Per-launch events add up to the GEMM time only while launches run one after the other: the pass
    # that records them keeps the matrices in one lane (a small model's matrices otherwise run as two
    # lanes on two streams, whose launches overlap).
    lanes_saved = plan.LANES
    if launch_events and not use_graph:
        plan.LANES = "1"
    try:
        return _run_optimizer_workload(muon_amd, engine, name, steps, warmup, seed, ns_variant, use_graph,
                                       realloc_grads, launch_events)
    finally:
        plan.LANES = lanes_saved


def _run_optimizer_workload(muon_amd, engine, name, steps, warmup, seed, ns_variant, use_graph, realloc_grads,
                            launch_events):
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
    # --realloc-grads: what a training loop with zero_grad(set_to_none=True) does to the optimizer.
    # Every gradient sits at another address than the step before, so the descriptor tables are
    # re-validated and uploaded again inside the timed region.  Two resident sets alternate, so no
    # copy or allocation of the gradients themselves is timed.
    spare = [p.grad.clone() for p in pm + pa] if realloc_grads else None

    def one_step():
        if spare is not None:
            for i, p in enumerate(pm + pa):
                p.grad, spare[i] = spare[i], p.grad
        opt.step()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()

    # timed region: exactly `steps` steps back to back, one synchronisation on either side; a pair
    # of HIP events on the launch stream brackets every kernel launch inside it (recording them
    # costs the host a few microseconds per launch, which a step of a small model notices:
    # launch_events=False times the same region without them)
    engine.PROFILE = None if (use_graph or not launch_events) else []      # a replayed graph has no per-launch events
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
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
    assert all(torch.isfinite(p).all() for p in pm[:2] + pa[:2])
    del opt, pm, pa, spare
    torch.cuda.empty_cache()
    return dict(ms_per_step=total_ms / steps, per_label=per_label, muon_elements=n_m, adam_elements=n_a,
                f_sym=fs, f_dense=fd)


def run_backward_overlap(name, iters=10, warmup=3, tokens=65536, seed=4321):
    """A training iteration = zero_grad, a synthetic backward, step(), with and without
    overlap_backward.  The backward is what autograd does for the weights of linear layers fed a
    batch of `tokens` tokens under bf16 autocast: one weight-gradient product x^T . dy per Muon
    matrix (for a conv filter, of its flattened form), an elementwise gradient for the Adam tensors.
    Reported per mode: the whole iteration and the step() call alone (HIP events on the launch
    stream; the work the hooks move out of step() runs inside the iteration either way)."""
    import muon_amd

    muon, adam, _, _, _ = workload_shapes(name)
    dev = torch.device("cuda:0")
    out = {"backward": f"synthetic: weight-gradient products of a {tokens}-token batch, bf16 autocast", "iters": iters}
    for mode in ("off", "on"):
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        pm = [torch.nn.Parameter(torch.randn(*shape, device=dev, generator=gen) * 0.02)
              for shape, count in muon for _ in range(count)]
        pa = [torch.nn.Parameter(torch.randn(*shape, device=dev, generator=gen) * 0.02)
              for shape, count in adam for _ in range(count)]
        xs, dys, by_width = [], [], {}
        for p in pm:                              # one input / output gradient per width, shared
            r, c = mat2d(tuple(p.shape))
            for w in (r, c):
                if w not in by_width:
                    by_width[w] = (torch.randn(tokens, w, device=dev, generator=gen) * 1e-2).bfloat16()
            xs.append(by_width[r])
            dys.append(by_width[c])
        coef = [torch.randn_like(p) * 1e-3 for p in pa]
        opt = muon_amd.SingleDeviceMuonWithAuxAdam([
            dict(params=pm, use_muon=True, lr=0.02, momentum=0.95, weight_decay=0.01),
            dict(params=pa, use_muon=False, lr=3e-4, betas=(0.9, 0.95), eps=1e-10, weight_decay=0.01)],
            overlap_backward=(mode == "on"))

        def iteration(ev=None):
            opt.zero_grad(set_to_none=True)
            with torch.autocast("cuda", dtype=torch.bfloat16):
                loss = sum(((x @ p.reshape(x.shape[1], -1)) * dy).sum() for p, x, dy in zip(pm, xs, dys))
            loss = loss + sum((p * c).sum() for p, c in zip(pa, coef))
            loss.backward()
            if ev is not None:
                ev[0].record()
            opt.step()
            if ev is not None:
                ev[1].record()

        for _ in range(warmup):
            iteration()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        t0 = time.perf_counter()
        for ev in evs:
            iteration(ev)
        torch.cuda.synchronize()
        out[f"iteration_ms_overlap_{mode}"] = round((time.perf_counter() - t0) * 1e3 / iters, 3)
        out[f"step_ms_overlap_{mode}"] = round(sum(a.elapsed_time(b) for a, b in evs) / iters, 3)
        if mode == "on":
            eng = next(iter(opt._muon_engines.values()))
            out["matrices_staged_during_backward"] = len(eng._skip)
        assert all(torch.isfinite(p).all() for p in pm[:2] + pa[:2])
        del opt, pm, pa, xs, dys, coef, by_width
        torch.cuda.empty_cache()
    return out


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
    del out, G
    muon_amd.clear_engine_cache()
    torch.cuda.empty_cache()
    return dict(ms_per_step=total_ms / steps, per_label=per_label, muon_elements=32 * 4096 * 4096, adam_elements=0,
                f_sym=32 * f_sym(4096, 4096), f_dense=32 * f_dense(4096, 4096))


def roofline_object(workload, gemm_work, gemm_ms, gemm_n):
    traffic = GEMM_TRAFFIC_BYTES_PER_LAUNCH.get(workload)
    return {
        "bound": "mfma",
        "kernel": "ns_gemm_kernel (syrk + poly + update launches)",
        "achieved": round(gemm_work / gemm_ms / 1e9, 1),
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(gemm_work / gemm_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
        "traffic": traffic[0] if traffic else None,
        "traffic_source": (traffic[1] + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this "
                           "command; a profile-derived constant, not measured in this run)") if traffic else None,
        "launches": gemm_n,
        "avg_launch_ms": round(gemm_ms / gemm_n, 4),
        "flops_per_launch": gemm_work / gemm_n,
    }


def rounded(kernels):
    return {k: {kk: (round(vv, 4) if isinstance(vv, float) else vv) for kk, vv in v.items()} for k, v in kernels.items()}


SECONDARY_SEEDS = {"gpt2-124m": 1234 + 2, "conv": 1234 + 5}


def secondary(name, gates):
    """A further benchmark configuration measured in the same run, as a sub-object."""
    out = {"gates": correctness_gates(name)} if gates else {}
    if name == "ns32":
        r = run_ns32(3, 1, seed=1234 + 3)
    else:
        _, _, _, dsteps, dwarm = workload_shapes(name)
        r = run_optimizer_workload(name, dsteps, dwarm, seed=SECONDARY_SEEDS[name])
    _, gw, gms, gn = summarize_kernels(r["per_label"])
    if name != "ns32":
        out["torch_gpu_baseline_ms_per_step"] = torch_gpu_baseline(name, steps=3)["ms_per_step"]
    out.update({"ms_per_step": round(r["ms_per_step"], 3), "ns_tflops_sym": round(gw / gms / 1e9, 1),
                "ns_frac_of_peak": round(gw / gms / 1e9 / PEAK_BF16_TFLOPS, 4), "gemm_launches": gn,
                "avg_gemm_launch_ms": round(gms / gn, 4)})
    if name != "ns32":
        # the same steps without the per-launch events: what a training loop sees
        plain = run_optimizer_workload(name, dsteps, dwarm, seed=SECONDARY_SEEDS[name], launch_events=False)
        out["ms_per_step_with_launch_events"] = out["ms_per_step"]
        out["ms_per_step"] = round(plain["ms_per_step"], 3)
        g = run_optimizer_workload(name, dsteps, dwarm, seed=SECONDARY_SEEDS[name], use_graph=True)
        out["ms_per_step_graph_replay"] = round(g["ms_per_step"], 3)
    if name != "ns32":
        b = workload_bounds(name)
        if name == "conv":
            # every matrix is short: the whole step is HBM / latency bound
            bound_ms = b["hbm_ns_ms"] + b["hbm_elementwise_ms"]
            out["hbm_roofline"] = {
                "bound": "hbm", "algorithmic_bytes": b["ns_bytes"] + b["elementwise_bytes"],
                "what": "5*(6mn+8m^2) B per matrix + 24 B per Muon element + 28 B per Adam element",
                "achieved_gbs": round((b["ns_bytes"] + b["elementwise_bytes"]) / out["ms_per_step"] / 1e6, 1),
                "peak_gbs": PEAK_HBM_GBS}
            out["hbm_frac"] = round(bound_ms / out["ms_per_step"], 4)
        else:
            # MFMA-bound products + HBM-bound elementwise kernels, one after the other
            bound_ms = b["mfma_ms"] + b["hbm_elementwise_ms"]
            out["bound_parts_ms"] = {"mfma": round(b["mfma_ms"], 4), "hbm_elementwise": round(b["hbm_elementwise_ms"], 4)}
        out["bound_ms"] = round(bound_ms, 4)
        out["bound_frac"] = round(bound_ms / out["ms_per_step"], 4)
        r = run_optimizer_workload(name, dsteps, dwarm, seed=SECONDARY_SEEDS[name], realloc_grads=True, launch_events=False)
        out["ms_per_step_realloc_grads"] = round(r["ms_per_step"], 3)
    if name == "gpt2-124m":
        out["backward_overlap"] = run_backward_overlap(name)
    return out


def product_operators(gates):
    """The three products as operators of their own (ns_line_1 / ns_line_2 / ns_line_3, reference
    muon.py:420, 547, 705) on the shapes of the Llama-3-8B feed-forward matrices: checked against
    the oracle on a small ragged case first, then timed with HIP events (results written into
    buffers given by the caller, as the reference's iteration does, muon.py:789-794)."""
    import muon_amd
    from oracle import muon_oracle as O

    out = {}
    dev = torch.device("cuda:0")
    if gates:
        g = torch.Generator().manual_seed(99)
        X = (torch.randn(2, 200, 328, generator=g) * 0.05).bfloat16()
        S = O.ns_line_1(X)
        worst = 0.0
        for name, got, want in (
                ("ns_line_1", muon_amd.ns_line_1(X.to(dev)), S),
                ("ns_line_2", muon_amd.ns_line_2(S.to(dev), 2.0315, -4.7750), O.ns_line_2(S, 2.0315, -4.7750)),
                ("ns_line_3", muon_amd.ns_line_3(S.to(dev), X.to(dev), 3.4445), O.ns_line_3(S, X, 3.4445))):
            d = (got.double().cpu() - want.double()).abs()
            step = 2.0 ** -7 * want.double().abs() + 1e-4            # one bf16 step at the value
            if not (d <= step).all():
                sys.exit(f"bench.py: correctness gate failed before timing: {name} is more than one bf16 step from the oracle")
            worst = max(worst, float((d / step).max()))
        out["gate_max_bf16_steps_from_oracle"] = round(worst, 3)
    b, m, n = 16, 4096, 14336
    X = (torch.randn(b, m, n, device=dev) * 0.01).bfloat16()
    A = torch.empty(b, m, m, device=dev, dtype=torch.bfloat16)
    B = torch.empty_like(A)
    C = torch.empty_like(X)
    calls = (("ns_line_1", lambda: muon_amd.ns_line_1(X, out=A), b * m * (m + 1) * n),
             ("ns_line_2", lambda: muon_amd.ns_line_2(A, 2.0315, -4.7750, out=B), b * m * m * (m + 1)),
             ("ns_line_3", lambda: muon_amd.ns_line_3(B, X, 3.4445, out=C), 2 * b * m * m * n))
    out["shape"] = f"{b} x ({m} x {n}), bf16; flops: the minimum given symmetry"
    for name, call, flops in calls:
        call()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 3
        out[name] = {"ms": round(ms, 3), "tflops": round(flops / ms / 1e9, 1),
                     "frac_of_peak": round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    del X, A, B, C
    muon_amd.clear_engine_cache()
    torch.cuda.empty_cache()
    return out


# ------------------------------------------------------------------------------------------
# Library baseline on the same GPU: the reference's step written with torch operations (bf16
# torch.matmul = rocBLAS / hipBLASLt for the Newton-Schulz products, one parameter after the other,
# nothing fused) -- what the reference's algorithm costs on this GPU without this library.
# ------------------------------------------------------------------------------------------
def torch_gpu_baseline(name, steps=2, warmup=1):
    muon, adam, gstd, _, _ = workload_shapes(name)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(77)
    a, b, c = 3.4445, -4.7750, 2.0315                          # muon.py:276
    lr, wd, beta = 0.02, 0.01, 0.95

    def ns5(G):                                                # muon.py:265-291
        X = G.bfloat16()
        tall = G.size(-2) > G.size(-1)
        if tall:
            X = X.mT
        X = X / (X.norm(dim=(-2, -1), keepdim=True) + 1e-7)
        for _ in range(5):
            A = X @ X.mT
            B = b * A + c * A @ A
            X = a * X + B @ X
        return X.mT if tall else X

    pm = [torch.randn(*shape, device=dev, generator=gen) * 0.02 for shape, count in muon for _ in range(count)]
    pa = [torch.randn(*shape, device=dev, generator=gen) * 0.02 for shape, count in adam for _ in range(count)]
    gm = [torch.randn_like(p) * gstd for p in pm]
    ga = [torch.randn_like(p) * gstd for p in pa]
    mom = [torch.zeros_like(p) for p in pm]
    ea, eas = [torch.zeros_like(p) for p in pa], [torch.zeros_like(p) for p in pa]

    def step(t):
        for p, g0, m in zip(pm, gm, mom):                      # muon.py:8-15, 97-99
            g = g0.clone()                                     # the reference overwrites p.grad; keep ours for the next step
            m.lerp_(g, 1 - beta)
            u = g.lerp_(m, beta)
            if u.ndim == 4:
                u = u.view(len(u), -1)
            u = ns5(u)
            u *= max(1, g.size(-2) / g.size(-1)) ** 0.5
            p.mul_(1 - lr * wd)
            p.add_(u.reshape(p.shape), alpha=-lr)
        for p, g, m, v in zip(pa, ga, ea, eas):                # muon.py:104-109, 257-258
            m.lerp_(g, 0.1)
            v.lerp_(g.square(), 0.05)
            upd = (m / (1 - 0.9 ** t)) / ((v / (1 - 0.95 ** t)).sqrt() + 1e-10)
            p.mul_(1 - 3e-4 * wd)
            p.add_(upd, alpha=-3e-4)

    with torch.no_grad():
        for t in range(1, warmup + 1):
            step(t)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for t in range(warmup + 1, warmup + steps + 1):
            step(t)
        torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    del pm, pa, gm, ga, mom, ea, eas
    torch.cuda.empty_cache()
    return dict(ms_per_step=round(ms, 3), steps=steps,
                what="the reference step (muon.py:8-15, 97-109, 257-258, 265-291) as torch operations on this GPU: "
                     "bf16 torch.matmul for the Newton-Schulz products, per parameter, unfused")


# ------------------------------------------------------------------------------------------
# CPU baseline: the oracle restatement of the reference on the host cores, bounded sample
# ------------------------------------------------------------------------------------------
def host_threads():
    """Threads for the host-side legs: every core the process may use (bounded by the
    OMP_NUM_THREADS of the environment when that is set, as on a host whose cores are shared)."""
    n = os.cpu_count() or 1
    if hasattr(os, "sched_getaffinity"):
        n = min(n, len(os.sched_getaffinity(0)))
    env = os.environ.get("OMP_NUM_THREADS", "")
    if env.isdigit() and int(env) > 0:
        n = min(n, int(env))
    return n


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(name, budget_s=25.0):
    from oracle import muon_oracle as O
    cores = host_threads()
    torch.set_num_threads(cores)
    muon, adam, gstd, _, _ = workload_shapes(name)
    torch.manual_seed(4321)
    total_ms, parts, t_start = 0.0, [], time.perf_counter()

    def timed_step(opt):
        opt.step()                      # warm-up: thread pool, allocator, lazy state
        t0 = time.perf_counter()
        opt.step()
        return (time.perf_counter() - t0) * 1e3

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
        ms = timed_step(O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p], use_muon=True, lr=0.02, weight_decay=0.01)]))
        total_ms += ms * count
        parts.append(f"muon {count}x{tuple(shape)}@{ms:.0f}ms")
    # Adam: one slab of at most 4096 rows of each distinct shape, scaled by element count
    for shape, count in adam:
        rows = min(shape[0], 4096)
        sl = (rows,) + tuple(shape[1:])
        p = torch.nn.Parameter(torch.randn(*sl) * 0.02)
        p.grad = torch.randn(*sl) * gstd
        ms = timed_step(O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p], use_muon=False, weight_decay=0.01)]))
        ms *= shape[0] / rows
        total_ms += ms * count
        parts.append(f"adam {count}x{tuple(shape)}@{ms:.1f}ms (from a {rows}-row slab)")
    skipped = any("skipped" in s for s in parts)
    return dict(value=None if skipped else round(total_ms, 1), unit="ms/step", cores=cores, cpu=cpu_model(), kind="port",
                sample="one warmed-up oracle step per distinct Muon shape and per <=4096-row slab of each Adam shape, "
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
    ap.add_argument("--realloc-grads", action="store_true",
                    help="give every parameter a gradient at a new address each step (as zero_grad("
                         "set_to_none=True) does), so that re-binding the descriptor tables is timed")
    ap.add_argument("--no-gates", action="store_true", help="skip the correctness gates (profiling runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-torch-baseline", action="store_true",
                    help="skip timing the same step written with torch operations on this GPU")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations (GPT-2, ns32, conv)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="first run one plain 1 GiB device-to-device copy kernel (a known-size reference "
                         "for scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the Muon update shards "
                 "by matrix across ranks, which is not part of this library). Run with --gpus 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X GPU")
    gates = None if args.no_gates else correctness_gates(args.workload)
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
            "gates": gates,
            "roofline": roofline_object("ns32", gemm_work, gemm_ms, gemm_n),
            "ns": {"tflops_sym_whole_call": round(res["f_sym"] / res["ms_per_step"] / 1e9, 1),
                   "tflops_dense_equiv_whole_call": round(res["f_dense"] / res["ms_per_step"] / 1e9, 1)},
            "kernels": rounded(kernels),
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
                                 use_graph=args.graph, realloc_grads=args.realloc_grads)
    grads = "new address every step" if args.realloc_grads else "resident, same addresses every step"
    if args.graph:
        print(json.dumps({"metric": f"muon_step_ms_{args.workload}", "value": round(res["ms_per_step"], 3),
                          "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warmup,
                          "ms_per_step": round(res["ms_per_step"], 3), "higher_is_better": False,
                          "config": {"workload": args.workload, "ns_variant": args.ns_variant, "launch": "hip graph replay",
                                     "gradients": grads}}))
        return
    kernels, gemm_work, gemm_ms, gemm_n = summarize_kernels(res["per_label"])
    ew_bytes = sum(w for l, (w, ms, n) in res["per_label"].items() if not l.startswith("ns_gemm"))
    ew_ms = sum(ms for l, (w, ms, n) in res["per_label"].items() if not l.startswith("ns_gemm"))
    alg_bytes = (res["muon_elements"] * 24 + res["adam_elements"] * 28) * steps
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
                   "ns_variant": args.ns_variant, "gradients": grads},
        "gates": gates,
        "roofline": roofline_object(args.workload, gemm_work, gemm_ms, gemm_n),
        "ns": {
            "ns_ms_per_step": round(gemm_ms / steps, 3),
            "tflops_sym": round(res["f_sym"] * steps / gemm_ms / 1e9, 1),
            "tflops_dense_equiv": round(res["f_dense"] * steps / gemm_ms / 1e9, 1),
        },
        "elementwise": {
            "ms_per_step": round(ew_ms / steps, 3),
            "launched_gbs": round(ew_bytes / ew_ms / 1e6, 1),
            "algorithmic_gbs": round(alg_bytes / ew_ms / 1e6, 1),
            "frac_of_hbm_peak_algorithmic": round(alg_bytes / ew_ms / 1e6 / PEAK_HBM_GBS, 4),
        },
        "kernels": rounded(kernels),
    }
    if args.workload != "llama3-8b" and not args.realloc_grads:
        # a small model's step is short enough for the host cost of the launch events to show
        plain = run_optimizer_workload(args.workload, steps, warmup, seed=1234 + 4, ns_variant=args.ns_variant,
                                       launch_events=False)
        line["ms_per_step_without_launch_events"] = round(plain["ms_per_step"], 3)
    if not args.no_extra and args.workload == "llama3-8b":
        line["gpt2_124m"] = secondary("gpt2-124m", not args.no_gates)
        line["ns32"] = secondary("ns32", not args.no_gates)
        line["conv"] = secondary("conv", not args.no_gates)
        line["product_operators"] = product_operators(not args.no_gates)
    if not args.no_torch_baseline:
        line["torch_gpu_baseline"] = torch_gpu_baseline(args.workload)
        line["torch_gpu_baseline"]["speedup"] = round(line["torch_gpu_baseline"]["ms_per_step"] / res["ms_per_step"], 2)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.workload)
        if line["cpu_baseline"]["value"]:
            line["cpu_baseline"]["gpu_speedup"] = round(line["cpu_baseline"]["value"] / res["ms_per_step"], 1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
