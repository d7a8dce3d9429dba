"""Benchmark of the fused learned-optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gpt2s|cfg1|vit_velo|llama_adafac|stress_velo|stress_celo2|conv_celo2|llama_celo2|stream_ceiling|matrix_ceiling] [--fused-only]

Workload (default): BASELINE config 2 -- ELO-CELO2 on a GPT-2-small-shaped fp32 parameter set
(98 tensors, 124 355 328 parameters), synthetic per-tensor Gaussian gradients with log-uniform
scale in [1e-5, 1e-2], random-init CELO2MLP, everything resident in HBM before timing starts.

A *step* of the metric is one whole ``optimizer.step()``: the single C-ABI call
``pylo_mi355_celo2_step`` (gradient statistics, accumulator updates, features, MLP, raw step for the
2-D tensors, AdamW for the 1-D tensors), Newton-Schulz on every raw step, and the finishing pass that
normalises the steps and updates the matrices.  ``value`` is parameters updated per second by that.
The HBM-bound part -- the C-ABI call -- is timed inside the same steps with HIP events recorded by the
library on the launch stream (``fused_pass``, ``roofline``), and once more alone, back to back; VeLO on
the ViT-B/16 set and AdafacLO on the Llama-1.1B set are measured after it (``velo_vitb16``,
``llama_adafac``).

Prints ONE JSON line.
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
B_P0, B_STATS, B_APPLY = 4, 24, 44   # algorithmic bytes per element of a >=2-D tensor, per pass
B_ADAM = 44                    # 1-D AdamW branch: read g,p,m0..2,rms; write m0..2,rms,p


def gpt2_small_shapes():
    shapes = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (768, 768), (768,), (768,), (768, 3072), (3072, 768)]
    return shapes


def cfg1_shapes():
    return [(1024, 1024), (1024,)]


def vit_b16_shapes():
    """BASELINE config 3 (VeLO): ViT-B/16, 100 tensors, 86 481 408 elements."""
    shapes = [(768, 3, 16, 16), (1, 1, 768), (197, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (768, 768), (768,), (768,), (768, 3072), (3072, 768)]
    return shapes + [(768, 1000)]


def resnet50_shapes():
    """Not a BASELINE configuration: ResNet-50, 161 tensors, 25 557 032 elements, 11.3 M of them in 3 x 3 kernels --
    the tensors with more than two dims that ELO-CELO2 orthogonalises, normalises and applies per slice."""
    shapes = [(64, 3, 7, 7), (64,), (64,)]
    inplanes = 64
    for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            shapes += [(planes, inplanes, 1, 1), (planes,), (planes,), (planes, planes, 3, 3), (planes,), (planes,),
                       (planes * 4, planes, 1, 1), (planes * 4,), (planes * 4,)]
            if b == 0:
                shapes += [(planes * 4, inplanes, 1, 1), (planes * 4,), (planes * 4,)]
            inplanes = planes * 4
    return shapes + [(1000, 2048), (1000,)]


def llama_1b_shapes(layers=22):
    """BASELINE config 4 (AdafacLO): Llama-1.1B, 200 tensors, 1 100 046 336 elements."""
    shapes = [(32000, 2048)]
    for _ in range(layers):
        shapes += [(2048,), (2048, 2048), (2048, 256), (2048, 256), (2048, 2048), (2048,),
                   (2048, 5632), (2048, 5632), (5632, 2048)]
    return shapes + [(32000, 2048)]


def stress_shapes(n_tensors=3000, seed=11, embedding=(32000, 4096)):
    """BASELINE config 5: tensors of 1 .. 65 536 elements drawn log-uniform, 1-D and 2-D with odd dims mixed, plus one
    32000 x 4096 embedding (the generator of tests/test_many_tensors_gpu.py)."""
    import math

    import torch

    gen = torch.Generator().manual_seed(seed)
    shapes = [(37, 4099), (4099, 37)]
    while len(shapes) < n_tensors:
        n = max(int(math.exp(float(torch.rand((), generator=gen)) * math.log(65536.0))), 1)
        if float(torch.rand((), generator=gen)) < 0.4:
            shapes.append((n,))
        else:
            r = max(1, int(math.exp(float(torch.rand((), generator=gen)) * math.log(n))))
            shapes.append((r, max(1, n // r)))
    return shapes + [embedding]


def layer_sample_shapes():
    return [(768,), (768,), (768, 2304), (768, 768), (768,), (768,), (768, 3072), (3072, 768)]


def make_inputs(shapes, device, seed=0):
    import torch

    gen = torch.Generator(device="cpu").manual_seed(seed)
    scales = [10 ** (-5 + 3 * float(torch.rand((), generator=gen))) for _ in shapes]
    ggen = torch.Generator(device=device).manual_seed(seed + 1)
    params, grads = [], []
    for s, sc in zip(shapes, scales):
        params.append(torch.nn.Parameter(torch.randn(s, generator=ggen, device=device) * 0.02))
        grads.append(torch.randn(s, generator=ggen, device=device) * sc)
    return params, grads


def cpu_baseline(steps=14):
    """The oracle (CPU restatement of the reference's naive PyTorch path) on one transformer
    layer of the same workload, host cores of this box."""
    import torch

    from oracle import pylo_oracle as O
    from pylo_amd.models import CELO2MLP

    shapes = layer_sample_shapes()
    torch.manual_seed(1)
    net = CELO2MLP()
    params, grads = make_inputs(shapes, "cpu", seed=3)
    params = [p.detach().clone() for p in params]
    orc = O.EloCelo2Oracle(params, net.state_dict(), lr=3.16e-4, adam_lr_mult=20.0)
    n = sum(p.numel() for p in params)
    t_fused = t_all = 0.0
    for it in range(steps + 1):
        orc.finish_seconds = 0.0
        t0 = time.perf_counter()
        orc.step(grads)
        dt = time.perf_counter() - t0
        if it > 0:
            t_all += dt
            t_fused += dt - orc.finish_seconds
    return {
        "value": n * steps / t_all, "unit": "params/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle (torch-CPU restatement of ELO_CELO2_naive) on one GPT-2-small layer "
                  f"({n} params, {steps} whole steps after 1 warm-up: accumulators, features, MLP, AdamW, "
                  f"Newton-Schulz, normalise, apply); without Newton-Schulz/normalise/apply "
                  f"{n * steps / t_fused:.3e} params/s",
        "os_cpu_count": os.cpu_count(),
    }


def ns_flops(shapes, iters=5):
    """fp32 FLOPs of the Newton-Schulz iterations of one step (pylo/optim/CELO2_naive.py:59-73): per iteration
    and matrix with small dim m and large dim n, A = X X^T (2 m^2 n), (c2 A + c1 I) A (2 m^3), (B + c0 I) X (2 m^2 n)."""
    total = 0.0
    for s in shapes:
        if len(s) == 2:
            m, n = min(s), max(s)
            total += iters * (4.0 * m * m * n + 2.0 * m ** 3)
    return total


def ns_chains(iters):
    """The chain lengths the library uses for `iters` iterations (pylo_mi355.hip, ns_chains): pairs by default,
    PYLO_MI355_NS_CHAINS / PYLO_MI355_NS_PAIRS=0 in the environment, chains of one on the fp32 kernels."""
    if os.environ.get("PYLO_MI355_NS_PAIRS", "1") == "0" or os.environ.get("PYLO_MI355_NS_F32") == "1":
        return [1] * iters
    try:
        given = [int(v) for v in os.environ.get("PYLO_MI355_NS_CHAINS", "").split(",") if v]
    except ValueError:
        given = []
    if given and min(given) >= 1 and sum(given) == iters:
        return given
    return [2] * (iters // 2) + [1] * (iters % 2)


def ns_flops_executed(shapes, iters=5, tile=128):
    """FLOPs (fp32 multiply-adds x 2) that the library's kernels execute: symmetric m x m results on the 64 x 64
    blocks on and above the diagonal only (whole 128 x 128 tiles above it, three quadrants of those on it), and iterations in chains that share one Gram product and one update: a chain of L
    iterations is one Gram product, 4 L - 3 products of m x m matrices (L x Poly, 2 (L - 1) x Prod, (L - 1) x
    ProdA) and one update."""
    chains = ns_chains(iters)
    total = 0.0
    for s in shapes:
        if len(s) == 2:
            m, n = min(s), max(s)
            nt = -(-m // tile)
            # tiles on and above the diagonal; on a diagonal tile the quadrant below the diagonal is not computed
            upper = (nt * (nt + 1) / 2 - nt / 4) * tile * tile
            total += len(chains) * (2.0 * upper * n + 2.0 * m * m * n) + sum(4 * L - 3 for L in chains) * 2.0 * upper * m
    return total


def whole_step_object(whole_ms, finish_ms, n_params, flops, flops_exec):
    """The matrix-pipe part of the step against the peak of the pipe it runs on.  By default the products run
    on the fp16 matrix instructions with every fp32 operand split into two fp16 planes (scaled by a power of
    two): three fp16 products per fp32 product, so the executed work is 3 x the fp32 FLOPs against the
    2.5 PFLOP/s of dense fp16;
    PYLO_MI355_NS_F32=1 runs them on the fp32 matrix instructions (157.3 TFLOP/s).  `achieved` counts the FLOPs
    the kernels execute (the symmetric halves they skip earn nothing); by the reference's full fp32 products the
    same time is `nominal_fp32_TFLOPs`."""
    f32 = os.environ.get("PYLO_MI355_NS_F32") == "1"
    t = finish_ms * 1e-3
    mult, peak = (1.0, 157.3) if f32 else (3.0, 2500.0)
    return {
        "ms": whole_ms, "params_per_sec": n_params / (whole_ms * 1e-3), "finish_ms": finish_ms,
        "newton_schulz_TFLOP": flops / 1e12, "newton_schulz_TFLOP_executed": flops_exec / 1e12,
        "roofline": {"bound": "mfma",
                     "kernel": ("k_ns_gemm (fp32 matrix instructions)" if f32 else
                                "k_ns_hf_gemm (fp16 matrix instructions, 3 products per fp32 product)")
                               + " + finishing pass",
                     "achieved": mult * flops_exec / t / 1e12, "peak": peak, "unit": "TFLOP/s",
                     "frac": mult * flops_exec / t / 1e12 / peak,
                     "fp32_equivalent_TFLOPs": flops_exec / t / 1e12,
                     "nominal_fp32_TFLOPs": flops / t / 1e12,
                     # the same fp32 products in the work units of the three-plane bf16 scheme these kernels ran
                     # on before (six 16-bit products per fp32 product): comparable with earlier lines, not a
                     # rate the pipe executes
                     "frac_in_six_product_units": None if f32 else 6.0 * flops_exec / t / 1e12 / peak,
                     "traffic": None},
    }


def traffic_from_profile(fname, kernel):
    """HBM bytes per launch of `kernel` as the counter summary under profiles/ states them
    (a line `traffic_bytes_per_launch <kernel> = <bytes>`); None when the file does not hold it."""
    import re

    try:
        text = open(os.path.join(ROOT, "profiles", fname)).read()
    except OSError:
        return None
    m = re.search(r"^traffic_bytes_per_launch\s+%s\s*=\s*([0-9.eE+]+)" % re.escape(kernel), text, re.M)
    return float(m.group(1)) if m else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="gpt2s", choices=["gpt2s", "cfg1", "vit_velo", "llama_adafac", "stress_velo", "stress_celo2", "conv_celo2", "llama_celo2", "stream_ceiling", "matrix_ceiling"])
    ap.add_argument("--fused-only", action="store_true",
                    help="loop the C-ABI call alone (no Newton-Schulz / apply), e.g. under rocprofv3")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra-workloads", action="store_true",
                    help="skip the VeLO / AdafacLO sub-objects of the default line")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a 1 GiB device-to-device tensor copy (3x) so that a counter profile of "
                         "this command holds a kernel of known HBM traffic to scale FETCH_SIZE/WRITE_SIZE by")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import numpy as np
    import torch

    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    if a.workload in ("conv_celo2", "llama_celo2"):
        print(json.dumps(conv_workload(a.steps, a.warmup, a.workload)))
        return
    if a.workload in ("stress_velo", "stress_celo2"):
        print(json.dumps(stress_workload(a.workload, a.steps, a.warmup)))
        return
    if a.workload in ("vit_velo", "llama_adafac"):
        print(json.dumps(other_workload(a.workload, a.steps, a.warmup)))
        return
    if a.workload == "stream_ceiling":
        return stream_ceiling(a)
    if a.workload == "matrix_ceiling":
        return matrix_ceiling(a)
    dev = torch.device("cuda:0")
    shapes = gpt2_small_shapes() if a.workload == "gpt2s" else cfg1_shapes()
    torch.manual_seed(1)
    net = CELO2MLP()
    params, grads = make_inputs(shapes, dev)
    for p, g in zip(params, grads):
        p.grad = g
    opt = ELO_CELO2_CUDA(params, lr=3.16e-4, weight_decay=0.1, adam_lr_mult=20.0, network=net, hf_key=None)
    n_params = sum(p.numel() for p in params)
    n2d = sum(p.numel() for p in params if p.dim() >= 2)
    n1d = n_params - n2d
    bytes_fused = n2d * (B_P0 + B_STATS + B_APPLY) + n1d * B_ADAM

    if a.calib_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)                      # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    plan = None

    def fused_loop(k):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(k):
            opt.fused_step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / k

    if a.fused_only:
        for _ in range(a.warmup):
            opt.fused_step()
        ms = fused_loop(a.steps)
        print(json.dumps({"metric": "fused C-ABI call alone", "ms_per_step": ms, "steps": a.steps, "warmup": a.warmup,
                          "hbm_roofline_frac_fused_path": bytes_fused / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}))
        return

    # 1) the timed region: K whole optimizer steps.  step() is fused_step() + finish_step(); they are called one
    #    after the other here so that events on the launch stream can mark where one ends.  The library records
    #    its own HIP events around every launch of the C-ABI call during these same steps.
    for _ in range(a.warmup):
        opt.step()
    plan = opt._plan
    names = plan.launch_names()
    plan.timing_begin(a.steps)
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(a.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(a.steps):
        marks[k][0].record()
        tensors = opt.fused_step()
        marks[k][1].record()
        opt.finish_step(tensors)
        marks[k][2].record()
    torch.cuda.synchronize()
    whole_ms = (time.perf_counter() - t0) * 1e3 / a.steps
    per = plan.timing_end()                       # (steps, launches) ms
    mean = per.mean(axis=0)
    fused_in_step_ms = float(np.mean([m[0].elapsed_time(m[1]) for m in marks]))
    finish_ms = float(np.mean([m[1].elapsed_time(m[2]) for m in marks]))
    # 2) the C-ABI call alone, back to back (no Newton-Schulz between two calls)
    fused_alone_ms = fused_loop(a.steps)

    flops = ns_flops(shapes)
    flops_exec = ns_flops_executed(shapes)
    elem = "k_celo2_elem" if "k_celo2_elem" in names else "k_celo2_apply"
    b_elem = (B_STATS + B_APPLY) if elem == "k_celo2_elem" else B_APPLY
    elem_ms = float(mean[names.index(elem)])
    elem_gbs = n2d * b_elem / (elem_ms * 1e-3) / 1e9
    fused_ms = float(per.sum(axis=1).mean())
    out = {
        "metric": "optimizer step ms + params updated/sec, % of MI355X HBM roofline (124M params)",
        "value": n_params / (whole_ms * 1e-3),
        "unit": "params/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": whole_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": ("ELO_CELO2 optimizer.step(), GPT-2-small fp32 parameter set (98 tensors)"
                                if a.workload == "gpt2s" else "ELO_CELO2 optimizer.step(), 1024x1024 + 1024"),
                   "params": n_params, "tensors": len(shapes),
                   "timed": "wall clock over `steps` whole optimizer steps (fused C-ABI call, Newton-Schulz, "
                            "finishing pass) between two device synchronisations; every parameter is updated "
                            "in every timed step"},
        # the HBM-bound part of the step: the one C-ABI call (gradient statistics, accumulators, features, MLP,
        # raw step; AdamW for the 1-D tensors), timed inside the same steps by the library's events
        "fused_pass": {
            "ms": fused_ms, "ms_by_stream_events_around_the_call": fused_in_step_ms,
            "ms_alone_back_to_back": fused_alone_ms,
            "hbm_algorithmic_GB": bytes_fused / 1e9,
            "hbm_GBps": bytes_fused / (fused_ms * 1e-3) / 1e9,
            "hbm_roofline_frac": bytes_fused / (fused_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "hbm_roofline_frac_alone_back_to_back": bytes_fused / (fused_alone_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "params_per_sec_through_the_pass": n_params / (fused_ms * 1e-3),
            "note": "updates the 1-D (AdamW) parameters and writes the raw steps of the matrices; the matrices "
                    "themselves are updated by the finishing pass after Newton-Schulz",
            "launches_per_step": len(names),
            "launch_ms": {nm: float(v) for nm, v in zip(names, mean)},
        },
        "hbm_roofline_frac_fused_path": bytes_fused / (fused_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        # which part of ms_per_step each roofline speaks for: `roofline` below (HBM) is the fused call's dominant
        # kernel, `whole_step.roofline` (matrix pipe) is Newton-Schulz and the finishing pass
        "share_of_step": {"fused_pass (hbm roofline)": fused_in_step_ms / whole_ms,
                          "newton_schulz + finishing pass (mfma roofline, whole_step.roofline)": finish_ms / whole_ms},
        # Newton-Schulz + normalise + apply
        "whole_step": whole_step_object(whole_ms, finish_ms, n_params, flops, flops_exec),
        "roofline": {"bound": "hbm", "kernel": elem, "achieved": elem_gbs, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": elem_gbs / HBM_PEAK_GBS,
                     "traffic": traffic_from_profile("celo2_fused_step_gpt2s_hbm_traffic.txt", elem) if a.workload == "gpt2s" else None,
                     "algorithmic_bytes_per_launch": n2d * b_elem, "avg_launch_ms": elem_ms},
    }
    del opt, params, grads, plan
    torch.cuda.empty_cache()
    if a.workload == "gpt2s" and not a.no_extra_workloads:
        out["velo_vitb16"] = other_workload("vit_velo", a.steps, a.warmup)
        torch.cuda.empty_cache()
        out["llama_adafac"] = other_workload("llama_adafac", max(5, a.steps // 5), max(2, a.warmup // 5))
        torch.cuda.empty_cache()
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


def stream_ceiling(a):
    """What the memory system delivers for the access mixes of the element passes, with nothing computed:
    the library's bare streaming kernel over arrays of the GPT-2-small matrices' size.  Not a benchmark of
    the optimizer; it is the yardstick the roofline fractions of its kernels are read against."""
    import ctypes as C

    import torch

    from pylo_amd import _lib

    lib = _lib.load()
    lib.pylo_mi355_stream_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p]
    dev = torch.device("cuda:0")
    n = 124318464
    src = torch.zeros(6 * n, device=dev)
    dst = torch.zeros(5 * n, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    out = {}
    for name, r, w in (("read6 (statistics pass)", 6, 0), ("read6 write5 (apply pass)", 6, 5), ("read1 write1 (copy)", 1, 1),
                       ("read1 (gradient pass)", 1, 0), ("write5", 1, 5)):
        for nt in (0, 1):
            call = lambda: _lib.check(lib.pylo_mi355_stream_probe(src.data_ptr(), dst.data_ptr(), n, r, w, nt, stream),
                                      "stream_probe")
            for _ in range(max(a.warmup, 3)):
                call()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(a.steps):
                call()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / a.steps
            out[f"{name}{', non-temporal' if nt else ''}"] = {"ms": ms, "GBps": (r + w) * 4.0 * n / ms / 1e6}
    print(json.dumps({"metric": "attainable_hbm_rate_by_access_mix", "unit": "GB/s", "n_gpus": 1, "steps": a.steps,
                      "warmup": a.warmup, "elements_per_array": n, "peak_GBps": HBM_PEAK_GBS, "mixes": out}))


def matrix_ceiling(a):
    """What the fp16 matrix pipe delivers for the instruction mix of the Newton-Schulz products: the library's
    bare matrix-pipe kernel (the update product's main loop, 128 x 256 tiles, reduction length 768) on planes of
    the GPT-2-small set's size, with the data path taken away in steps, on random data and on zeros (the pipe's
    power, and with it the clock, depends on the operands).  The yardstick next to the data sheet's 2.5 PFLOP/s."""
    import ctypes as C

    import torch

    from pylo_amd import _lib

    lib = _lib.load()
    lib.pylo_mi355_matrix_probe.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    dev = torch.device("cuda:0")
    rows_x, rows_b, k = 163840, 768, 768          # 125.8 M elements of X against a 768 x 768 matrix
    stream = torch.cuda.current_stream(dev).cuda_stream
    res = {}
    for data in ("random", "zeros"):
        gen = torch.Generator(device=dev).manual_seed(0)
        # random numbers around 1 (no NaN or infinity), as fp16 bit patterns
        def planes(n):
            if data == "zeros":
                return torch.zeros(n, device=dev, dtype=torch.float16)
            return (torch.randn(n, generator=gen, device=dev) * 0.5).to(torch.float16)
        x = planes(rows_x * k * 2)
        b = planes(rows_b * k * 2)
        out = torch.zeros((rows_x // 128) * (rows_b // 256) * 256, device=dev)
        for mode, name in ((0, "product loop"), (1, "LDS reads + matrix instructions"), (2, "matrix instructions only"),
                           (3, "product loop, 256 x 256 tiles by 512 threads"),
                           (4, "product loop, first operand straight into registers")):
            call = lambda: _lib.check(lib.pylo_mi355_matrix_probe(x.data_ptr(), rows_x, b.data_ptr(), rows_b, k, mode,
                                                                  out.data_ptr(), stream), "matrix_probe")
            for _ in range(max(a.warmup, 3)):
                call()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(a.steps):
                call()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / a.steps
            res[f"{name}, {data}"] = {"ms": ms, "PFLOPs": 6.0 * rows_x * rows_b * k / ms / 1e12}
        del x, b, out
    print(json.dumps({"metric": "attainable_fp16_matrix_rate", "unit": "PFLOP/s", "n_gpus": 1, "steps": a.steps,
                      "warmup": a.warmup, "tile": "128x256, 3 x v_mfma_f32_32x32x16_f16 per fp32 tile product",
                      "peak_PFLOPs": 2.5, "cases": res}))


def conv_workload(steps, warmup, which="conv_celo2"):
    """Whole ELO_CELO2 optimizer.step() on a parameter set that is not a BASELINE configuration.
    conv_celo2: ResNet-50 -- the fused element call (per-slice feature normalisers for the convolution kernels), then
    one finishing call in which every kernel's k x k slices are orthogonalised, normalised and applied by the
    per-slice launches and the one matrix by the tiled products.
    llama_celo2: the Llama-1.1B set of config 4 under ELO-CELO2 (matrices with a smaller dim of 2048, the two
    32000 x 2048 embeddings orthogonalised like the rest): how the products do on larger m."""
    import numpy as np
    import torch

    from pylo_amd import ELO_CELO2_CUDA
    from pylo_amd.models import CELO2MLP

    dev = torch.device("cuda:0")
    shapes = resnet50_shapes() if which == "conv_celo2" else llama_1b_shapes()
    label = "ResNet-50 parameter set" if which == "conv_celo2" else "Llama-1.1B parameter set"
    gen = torch.Generator(device=dev).manual_seed(1)
    params = [torch.nn.Parameter(torch.randn(s, generator=gen, device=dev) * 0.02) for s in shapes]
    for p in params:
        p.grad = torch.randn(p.shape, generator=gen, device=dev) * 1e-2
    torch.manual_seed(1)
    opt = ELO_CELO2_CUDA(params, lr=3e-4, weight_decay=0.1, network=CELO2MLP(), hf_key=None)
    for _ in range(max(warmup, 4)):
        opt.step()
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(steps):
        marks[k][0].record()
        tensors = opt.fused_step()
        marks[k][1].record()
        opt.finish_step(tensors)
        marks[k][2].record()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    n = sum(p.numel() for p in params)
    n_nd = sum(p.numel() for p in params if p.dim() > 2)
    return {"metric": "params_updated_per_sec (whole optimizer.step())", "value": n / (ms * 1e-3), "unit": "params/s",
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "newton_schulz_TFLOP": ns_flops(shapes) / 1e12, "newton_schulz_TFLOP_executed": ns_flops_executed(shapes) / 1e12,
            "config": {"workload": "ELO_CELO2 whole optimizer.step(), " + label, "params": n,
                       "tensors": len(shapes), "params_in_tensors_with_more_than_two_dims": n_nd},
            "fused_call_ms": float(np.mean([m[0].elapsed_time(m[1]) for m in marks])),
            "finishing_call_ms": float(np.mean([m[1].elapsed_time(m[2]) for m in marks])),
            "tensors_left_to_torch_products": sum(1 for i, (g, p, adam) in enumerate(opt._tensors())
                                                  if not adam and p.dim() >= 2 and not opt._ns_ok[i])}


def stress_workload(workload, steps, warmup):
    """Config 5 (3 000 small tensors + one 32000 x 4096 embedding, Student-t gradients): the fused VeLO step or the
    fused ELO-CELO2 element call.  What it measures is the multi-tensor launch table: how long the host takes to
    enqueue a step (argument table of 3 001 rows) against how long the GPU takes to run it, and the launches."""
    import torch

    from pylo_amd import ELO_CELO2_CUDA, VeLO_CUDA
    from pylo_amd.models import CELO2MLP, VeLOMLP, VeLORNN

    dev = torch.device("cuda:0")
    shapes = stress_shapes()
    gen = torch.Generator(device=dev).manual_seed(1)
    params = [torch.nn.Parameter(torch.randn(s, generator=gen, device=dev) * 0.02) for s in shapes]
    torch.manual_seed(2)
    t3 = torch.distributions.StudentT(torch.tensor(3.0, device=dev))
    for p in params:
        p.grad = t3.sample(p.shape) * 1e-3
    torch.manual_seed(1)
    if workload == "stress_velo":
        opt = VeLO_CUDA(params, lr=1e-3, num_steps=1000, rnn=VeLORNN(), mlp=VeLOMLP())
        loss = torch.tensor(1.0, device=dev)
        step = lambda: opt.step(loss)
        label = "VeLO fused step"
    else:
        opt = ELO_CELO2_CUDA(params, lr=3e-4, network=CELO2MLP(), hf_key=None)
        step = opt.step
        label = "ELO_CELO2 whole optimizer.step() (fused call, Newton-Schulz of every matrix incl. 32000 x 4096, update)"
    # (one call around the tenth in flight takes 0.1 s on the host, once; it is kept out of the timed region)
    for _ in range(max(warmup, 16)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    plan = opt._plan
    plan.timing_begin(steps)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    per = plan.timing_end()
    n = sum(p.numel() for p in params)
    ms = (t2 - t0) * 1e3 / steps
    extra = {}
    if workload == "stress_celo2":
        # the fused element call alone, and the same step with the 32000 x 4096 matrix in an is_embedding group
        # (AdamW, no Newton-Schulz on it): what the 3 000 small tensors cost by themselves
        extra["fused_call_ms"] = float(per.sum(axis=1).mean())
        del opt
        torch.cuda.empty_cache()
        opt2 = ELO_CELO2_CUDA([{"params": params[:-1]}, {"params": params[-1:], "is_embedding": True}], lr=3e-4,
                              network=CELO2MLP(), hf_key=None)
        for _ in range(max(warmup, 16)):
            opt2.step()
        torch.cuda.synchronize()
        t3a = time.perf_counter()
        for _ in range(steps):
            opt2.step()
        t3b = time.perf_counter()
        torch.cuda.synchronize()
        t3c = time.perf_counter()
        extra["embedding_as_adamw_group"] = {"ms_per_step": (t3c - t3a) * 1e3 / steps,
                                             "host_enqueue_ms_per_step": (t3b - t3a) * 1e3 / steps}
        n_mats = sum(1 for s_ in shapes if len(s_) == 2)
        extra["matrices_orthogonalised_by_library_kernels"] = n_mats
        extra["matrices_left_to_torch_products"] = sum(1 for i, s_ in enumerate(shapes[:-1]) if len(s_) == 2 and not opt2._ns_ok[i])
        plan = opt2._plan
    return {"metric": "params_updated_per_sec (fused step, C-ABI call)" if workload == "stress_velo" else
            "params_updated_per_sec (whole optimizer.step())", "value": n / (ms * 1e-3), "unit": "params/s",
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": f"{label}, stress set of {len(shapes)} tensors (3 000 of 1 - 65 536 elements, 1-D and odd "
                                   f"2-D, plus 32000 x 4096)", "params": n, "tensors": len(shapes)},
            "host_enqueue_ms_per_step": (t1 - t0) * 1e3 / steps, **extra,
            "sum_of_launch_intervals_ms": float(per.sum(axis=1).mean()),
            "launch_ms": {nm: float(v) for nm, v in zip(plan.launch_names(), per.mean(axis=0))}}


def other_workload(workload, steps, warmup):
    """VeLO on the ViT-B/16 set (config 3) or AdafacLO on the Llama-1.1B set (config 4): same JSON
    line, the whole optimizer step is the fused C-ABI call for these two optimizers."""
    import torch

    from pylo_amd import AdafacLO_CUDA, VeLO_CUDA
    from pylo_amd.models import MetaMLP, VeLOMLP, VeLORNN

    dev = torch.device("cuda:0")
    torch.manual_seed(1)
    if workload == "vit_velo":
        shapes = vit_b16_shapes()
        params, grads = make_inputs(shapes, dev)
        opt = VeLO_CUDA(params, lr=1e-3, num_steps=10000, rnn=VeLORNN(), mlp=VeLOMLP())
        loss = torch.tensor(2.0, device=dev)
        step = lambda: opt.step(loss)
        apply_kernel, stats_kernel = "k_velo_apply", "k_velo_stats"
        label = "VeLO fused step, ViT-B/16 fp32 parameter set (100 tensors)"
    else:
        shapes = llama_1b_shapes()
        params, grads = make_inputs(shapes, dev)
        grads = [g.bfloat16().float() for g in grads]
        opt = AdafacLO_CUDA(params, lr=1.0, network=MetaMLP(39, 32, 1))
        step = opt.step
        apply_kernel, stats_kernel = "k_adafac_apply", "k_adafac_stats"
        label = "AdafacLO fused step, Llama-1.1B fp32 parameter set (200 tensors)"
    for p, g in zip(params, grads):
        p.grad = g
    n_params = sum(p.numel() for p in params)
    n2d = sum(p.numel() for p in params if p.dim() >= 2)
    n1d = n_params - n2d
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    fused_ms = (time.perf_counter() - t0) * 1e3 / steps   # the timed region: K back-to-back steps
    plan = opt._plan
    plan.timing_begin(steps)                               # second pass: HIP events around every launch
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    per = plan.timing_end()
    names = plan.launch_names()
    mean = per.mean(axis=0)
    # 1-D tensors also carry the per-element accumulator fac_v: +3 reads in both passes, +3 writes
    bytes_fused = n2d * (B_P0 + B_STATS + B_APPLY) + n1d * (36 + 36 + 32)
    b_elem, b_vec = B_APPLY, 68
    if "k_velo_elem" in names:        # statistics and apply items of all tensors in one launch
        apply_kernel, b_elem, b_vec = "k_velo_elem", B_STATS + B_APPLY, 36 + 68
    k = names.index(apply_kernel)
    apply_gbs = (n2d * b_elem + n1d * b_vec) / (float(mean[k]) * 1e-3) / 1e9
    roof = {"bound": "hbm", "kernel": apply_kernel, "achieved": apply_gbs, "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": apply_gbs / HBM_PEAK_GBS,
            "traffic": traffic_from_profile("velo_fused_step_vitb16_kernel_trace_and_traffic.txt", apply_kernel) if workload == "vit_velo" else None,
            "algorithmic_bytes_per_launch": n2d * b_elem + n1d * b_vec, "avg_launch_ms": float(mean[k])}
    if workload == "llama_adafac":
        # The 16 -> 32 -> 32 -> 2 element MLP: 1 600 FMAs per element of a >= 2-D tensor.  By default its two
        # wide layers (1 536 FMAs) run on the fp16 matrix instructions with two-plane operands, three fp16
        # products per fp32 product, and the kernel is bound by its vector instructions (the splitting of the
        # activations is vector work; the matrix instructions run under it);
        # PYLO_MI355_ADAFAC_F32=1 runs the layers on the fp32 matrix instructions.
        t = float(mean[k]) * 1e-3
        f32 = os.environ.get("PYLO_MI355_ADAFAC_F32") == "1"
        fp32_tflops = n2d * 3200.0 / t / 1e12
        if f32:
            roof = {"bound": "mfma", "kernel": "k_adafac_apply_tile (fp32 matrix instructions)", "achieved": fp32_tflops,
                    "peak": 157.3, "unit": "TFLOP/s", "frac": fp32_tflops / 157.3}
        else:
            bf = n2d * 3 * 1536 * 2.0 / t / 1e12
            roof = {"bound": "mfma", "kernel": "k_adafac_apply_tile (fp16 matrix instructions, 3 products per fp32 product)",
                    "achieved": bf, "peak": 2500.0, "unit": "TFLOP/s", "frac": bf / 2500.0,
                    "fp32_equivalent_TFLOPs": fp32_tflops, "fp32_matrix_peak_TFLOPs": 157.3}
        roof.update({"traffic": None, "avg_launch_ms": float(mean[k]), "hbm_GBps": apply_gbs})
    out = {
        "metric": "params_updated_per_sec (fused step, C-ABI call)", "value": n_params / (fused_ms * 1e-3),
        "unit": "params/s", "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": fused_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": label, "params": n_params, "tensors": len(shapes), "launches_per_step": len(names)},
        "hbm_algorithmic_GB_per_step": bytes_fused / 1e9,
        "hbm_GBps_fused_path": bytes_fused / (fused_ms * 1e-3) / 1e9,
        "hbm_roofline_frac_fused_path": bytes_fused / (fused_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,

        "sum_of_launch_intervals_ms": float(per.sum(axis=1).mean()),
        "launch_ms": {nm: float(v) for nm, v in zip(names, mean)},
        "roofline": roof,
    }
    del opt, params, grads, plan
    return out


if __name__ == "__main__":
    main()
