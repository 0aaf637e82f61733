#!/usr/bin/env python3
"""Benchmark of the optimizer-step hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c1|c3|c3s|c3nc|c2l|adopt|ademamix|nadam] [--no-cpu] [--no-muon]
                    [--no-soap] [--no-8b] [--soap-products]

Default workload (the headline configuration, "c2"): LaProp with ecc="bf16+8" on a GPT-2-small-shaped parameter set
(147 tensors, 123,653,376 elements), fp32 parameters, bf16 gradients ~ N(0, 1e-3), synthetic data generated on the
device.  A "step" is one ``optimizer.step()`` over the whole set with the gradients already resident in HBM.

Prints ONE JSON line.  ``value`` is the wall-clock ms per step of ``optimizer.step()`` (host overhead included), the median
of ``--windows`` windows of ``--steps`` steps, each between two device synchronisations;
``roofline`` is computed from the fused kernel's own duration, measured with HIP events on the launch stream around
back-to-back launches of ``hb_fused_step``; ``cpu_baseline`` is the CPU oracle (an op-for-op restatement of the
reference's eager path) timed on this machine's host cores: the whole of configuration c2, three steps after a warm-up.
Beside the headline the line carries the reference's own micro-benchmark protocol (``adamw_reference_script``), Muon's
Newton-Schulz (``ns5``), SOAP (``soap``) and, when 200 GiB of device memory are free, the Llama-3-8B-shaped parameter set
under LaProp and under AdamW with MARS, caution, ECC states and ECC parameters (``llama8b``), each with its own roofline.
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "optimizer ms/step + achieved HBM GB/s (% of peak), 124M ECC LaProp; NS5 MFMA %"
HBM_PEAK_GBPS = 8000.0


def gpt2_small_shapes():
    """Benchmark configuration 2: 12 layers + final LN + token embedding, no position embedding (147 tensors)."""
    shapes = []
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]
    shapes += [(768,), (768,), (50257, 768)]
    return shapes


def llama8b_shapes(layers=32, vocab=128256):
    """Benchmark configuration 3: Llama-3-8B-shaped (291 tensors at 32 layers)."""
    shapes = []
    for _ in range(layers):
        shapes += [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336), (4096,), (4096,)]
    shapes += [(vocab, 4096), (vocab, 4096), (4096,)]
    return shapes


CONFIGS = {
    # name: (class, kwargs, shapes, grad dtype, grad std, algorithmic bytes per element, label)
    "c1": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01),
           [(1024, 1024), (1024,), (4096, 1024), (1024, 4096)], "float32", 1e-2, 28,
           "AdamW fp32, 4 tensors, 9.4M elements"),
    "c2": ("LaProp", dict(ecc="bf16+8"), gpt2_small_shapes(), "bfloat16", 1e-3, 22,
           "LaProp ecc=bf16+8, GPT-2-small-shaped 147 tensors, 123,653,376 elements, fp32 params, bf16 grads"),
    "c3": ("AdamW", dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"), llama8b_shapes(), "bfloat16", 1e-3, 26,
           "AdamW mars+caution ecc=bf16+8 param_ecc=bf16+8, Llama-3-8B-shaped 291 tensors, 8,030,261,248 elements"),
    "c3s": ("AdamW", dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8"), llama8b_shapes(4, 32064), "bfloat16", 1e-3, 26,
            "AdamW mars+caution ecc param_ecc, 4 Llama-3-8B layers + reduced vocab"),
    # the 8B-shaped parameter set without the second launch that caution needs, and under the optimizer of c2
    "c3nc": ("AdamW", dict(mars=True, ecc="bf16+8", param_ecc="bf16+8"), llama8b_shapes(), "bfloat16", 1e-3, 26,
             "AdamW mars ecc=bf16+8 param_ecc=bf16+8 (no caution), Llama-3-8B-shaped 291 tensors, 8,030,261,248 elements"),
    "c2l": ("LaProp", dict(ecc="bf16+8"), llama8b_shapes(), "bfloat16", 1e-3, 22,
            "LaProp ecc=bf16+8, Llama-3-8B-shaped 291 tensors, 8,030,261,248 elements, fp32 params, bf16 grads"),
    # the other fused first-order optimizers on the tensors of c2 (same roles and formats; AdEMAMix carries a third ECC state)
    "adopt": ("ADOPT", dict(ecc="bf16+8"), gpt2_small_shapes(), "bfloat16", 1e-3, 22, "ADOPT ecc=bf16+8 on the tensors of c2"),
    "ademamix": ("AdEMAMix", dict(ecc="bf16+8"), gpt2_small_shapes(), "bfloat16", 1e-3, 28, "AdEMAMix ecc=bf16+8 on the tensors of c2"),
    "nadam": ("NAdam", dict(ecc="bf16+8"), gpt2_small_shapes(), "bfloat16", 1e-3, 22, "NAdam ecc=bf16+8 on the tensors of c2"),
}  # fmt: skip


def cpu_baseline(cfg_name, total_elems):
    """The CPU oracle on a bounded sample of the same workload; returns the dict for the JSON line."""
    import torch

    from oracle import first_order as fo
    from oracle.rounding import TorchRounding

    cls, kwargs, shapes, gdt, gstd, _, _ = CONFIGS[cfg_name]
    if cfg_name in ("c3", "c3s", "c3nc", "c2l"):
        sample = [(1024, 4096), (1024, 4096), (4096,), (4096,), (2048, 4096)]
        what = "k/v projections, two norms and a [2048,4096] slice of one Llama-3-8B layer"
    else:
        sample = shapes
        what = "the full config (every tensor, every element)"
    n = sum(int(torch.Size(s).numel()) for s in sample)
    gen = torch.Generator().manual_seed(0)
    params = [torch.randn(s, generator=gen) * 0.02 for s in sample]
    kind = {"AdamW": "adam", "LaProp": "laprop", "ADOPT": "adopt", "AdEMAMix": "ademamix", "NAdam": "nadam"}[cls]
    orc = fo.FirstOrderOracle(kind, params, rounding=TorchRounding(), **kwargs)
    dt = getattr(torch, gdt)
    times = []
    for k in range(1, 5):
        grads = [(torch.randn(s, generator=gen) * gstd).to(dt) for s in sample]
        t0 = time.perf_counter()
        orc.step(grads)
        times.append(time.perf_counter() - t0)
        if sum(times) > 25.0 and len(times) >= 2:  # bounded: about half a minute of CPU work at most
            break
    per_step = statistics.median(times[1:])
    scaled_ms = per_step * 1e3 * total_elems / n
    return {
        "value": round(scaled_ms, 3),
        "unit": "ms/step",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{what}: {n} elements, median of {len(times) - 1} steps after 1 warm-up = {per_step * 1e3:.1f} ms, "
                  f"scaled linearly to {total_elems} elements; torch {torch.__version__} eager CPU ops in the reference's order",
        "elements_per_s": round(n / per_step, 1),
        # the lines of torch.__config__.parallel_info() that name the threading back end and its thread counts
        "parallel_info": "; ".join(ln.strip() for ln in torch.__config__.parallel_info().splitlines()
                                   if any(k in ln for k in ("ATen parallel backend", "get_num_threads", "max_threads", "num_interop"))),
    }  # fmt: skip


# hb::fused_step_kernel's HBM traffic per launch on config c2, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs scaled
# against a copy of known size (not measured in this run): the value and the file that documents it
C2_TRAFFIC_FROM_PROFILE = (2722.5e6, "profiles/fused_step_c2_hbm_traffic.txt")


def bench_first_order(cfg_name, steps, warmup, kernel_launches, rounding="philox", windows=5):
    """One first-order configuration: ``windows`` timed windows of ``steps`` calls of ``optimizer.step()`` each over the whole
    parameter set with the gradients resident in HBM (wall clock between two device synchronisations, host overhead included;
    the median window is reported, as the reference's benchmarks/bench_optimizer_step.py:66-81 does), then the kernel alone:
    HIP events on the launch stream around back-to-back ``hb_fused_step`` calls on the same descriptor.  Returns the fields of
    the JSON line."""
    import torch

    import heavyball_amd
    from heavyball_amd import _lib

    dev = torch.device("cuda:0")
    cls_name, kwargs, shapes, gdt, gstd, bytes_per_elem, label = CONFIGS[cfg_name]
    gdtype = getattr(torch, gdt)
    total = sum(int(torch.Size(s).numel()) for s in shapes)

    torch.manual_seed(0)
    params = []
    for s in shapes:
        p = torch.nn.Parameter(torch.randn(s, device=dev) * 0.02)
        p.grad_dtype = None
        params.append(p)
    opt = getattr(heavyball_amd, cls_name)(params, **kwargs)
    opt.rounding = rounding
    # gradient sets resident in HBM before the timed region, cycled.  Two even for the 8B-shaped set (16 GB each): with one set
    # every step would see the gradient of the step before, MARS' correction would vanish and caution's count pass would never
    # meet an element that is too close to call
    n_sets = 4 if total < 1_000_000_000 else 2
    grad_sets = [[(torch.randn(s, device=dev) * gstd).to(gdtype) for s in shapes] for _ in range(n_sets)]

    def one_step(k):
        gs = grad_sets[k % n_sets]
        for p, g in zip(params, gs):
            p.grad = g
        opt.step()

    for k in range(warmup):
        one_step(k)
    walls, issues = [], []
    for w in range(windows):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(steps):
            one_step(k)
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t0) * 1e3 / steps)
        issues.append((t1 - t0) * 1e3 / steps)
    ms_per_step = statistics.median(walls)
    host_ms = statistics.median(issues)  # the host's share: setting the gradients and issuing the step, without waiting for the device

    # kernel-only duration: HIP events on the launch stream around back-to-back launches of the same descriptor
    desc, _ = opt._last_launch
    L = _lib.lib()
    stream = torch.cuda.current_stream(dev)
    for _ in range(3):
        _lib.check(L.hb_fused_step(desc, stream.cuda_stream))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(kernel_launches):
        _lib.check(L.hb_fused_step(desc, stream.cuda_stream))
    e1.record(stream)
    torch.cuda.synchronize()
    kernel_ms = e0.elapsed_time(e1) / kernel_launches
    algo_bytes = bytes_per_elem * total
    achieved = algo_bytes / (kernel_ms * 1e-3) / 1e9
    roofline = {
        "bound": "hbm",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": C2_TRAFFIC_FROM_PROFILE[0] if cfg_name == "c2" else None,
        "algorithmic_bytes_per_launch": algo_bytes,
        "kernel": "hb::fused_step_kernel (all launches of one hb_fused_step call)",
    }
    if cfg_name == "c2":
        roofline["traffic_source"] = f"{C2_TRAFFIC_FROM_PROFILE[1]} (hardware counters of an earlier run of this command, not of this run)"
    del grad_sets, params
    return {
        "config": {"workload": label, "elements": total, "tensors": len(shapes), "rounding": opt.rounding, "name": cfg_name},
        "ms_per_step": round(ms_per_step, 4),
        "windows": windows,
        "ms_per_step_windows": [round(w, 4) for w in walls],
        "host_issue_ms_per_step": round(host_ms, 4),
        "kernel_ms": round(kernel_ms, 4),
        "elements_per_s": round(total / (ms_per_step * 1e-3), 1),
        "roofline": roofline,
    }


MFMA_BF16_PEAK_TFLOPS = 2500.0
C4_SHAPES = [(4096, 4096), (4096, 4096), (1024, 4096), (1024, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]


def ns5_flops(rows, cols):
    m, n = min(rows, cols), max(rows, cols)
    return 5.0 * (4.0 * m * m * n + 2.0 * m * m * m)


def bench_muon(steps=5, warmup=2):
    """Benchmark configuration 4: Muon (betas[0]=0.95, 5 Newton-Schulz iterations, bf16) on one Llama-3-8B layer's matrices.
    Returns ms/step of ``optimizer.step()`` and the achieved bf16 TFLOP/s of the Newton-Schulz part, counted on the
    algorithmic 5*(4 m^2 n + 2 m^3) FLOP per matrix and timed with HIP events around the hb_ns5 calls alone."""
    import ctypes

    import torch

    import heavyball_amd
    from heavyball_amd import _lib
    from heavyball_amd.muon import NS_COEFFS, ns_coefficients

    dev = torch.device("cuda:0")
    torch.manual_seed(1)
    params = [torch.nn.Parameter(torch.randn(s, device=dev) * 0.02) for s in C4_SHAPES]
    opt = heavyball_amd.Muon(params, betas=(0.95, 0.99))
    grads = [torch.randn(s, device=dev) * 1e-2 for s in C4_SHAPES]

    def one_step():
        for p, g in zip(params, grads):
            p.grad = g
        opt.step()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps

    # the other coefficient schedule: zeroth_power_mode "legacy_newtonschulz" gives square matrices the single triple
    # 3.4445 / -4.7750 / 2.0315 and one more input rounding; the non-square ones keep the per-iteration table
    import heavyball_amd.muon as muon_mod

    muon_mod.zeroth_power_mode = "legacy_newtonschulz"
    try:
        one_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            one_step()
        torch.cuda.synchronize()
        ms_step_legacy = (time.perf_counter() - t0) * 1e3 / 3
    finally:
        muon_mod.zeroth_power_mode = "newtonschulz"

    L = _lib.lib()
    stream = torch.cuda.current_stream(dev)
    arr = (ctypes.c_float * 15)(*ns_coefficients(NS_COEFFS))
    n = len(C4_SHAPES)
    rows = (ctypes.c_int64 * n)(*[r for r, _ in C4_SHAPES])
    cols = (ctypes.c_int64 * n)(*[c for _, c in C4_SHAPES])
    nb = ctypes.c_int64()
    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows, cols, ctypes.byref(nb)))
    ws = torch.empty(nb.value, dtype=torch.uint8, device=dev)
    outs = [torch.empty_like(g) for g in grads]
    gp = (ctypes.c_void_p * n)(*[g.data_ptr() for g in grads])
    op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    scale = (ctypes.c_float * n)(*[max(1, r / c) ** 0.5 for r, c in C4_SHAPES])
    base = (ctypes.c_int64 * n)(*([0] * n))

    def ns_all():
        _lib.check(L.hb_ns5_batched(n, gp, op, rows, cols, arr, 0, 1e-7, scale, _lib.RNG_PHILOX, 1, 1, base, ws.data_ptr(), ws.numel(),
                                    stream.cuda_stream))  # fmt: skip

    ns_all()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 3
    e0.record(stream)
    for _ in range(reps):
        ns_all()
    e1.record(stream)
    torch.cuda.synchronize()
    ns_ms = e0.elapsed_time(e1) / reps
    flops = sum(ns5_flops(r, c) for r, c in C4_SHAPES)
    tflops = flops / (ns_ms * 1e-3) / 1e12
    return {
        "workload": "Muon betas[0]=0.95, Newton-Schulz 5 iterations bf16, matrices [4096,4096]x2 [1024,4096]x2 [14336,4096]x2 [4096,14336], fp32 grads",
        "ms_per_step": round(ms_step, 3),
        "ms_per_step_legacy_schedule": round(ms_step_legacy, 3),
        "ns5_ms": round(ns_ms, 3),
        "roofline": {
            "bound": "mfma",
            "achieved": round(tflops, 1),
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
            "traffic": None,
            "algorithmic_flops_per_step": flops,
            "kernel": "hb::ns_gemm4_kernel (15 grouped launches over all matrices inside hb_ns5_batched, plus norm and conversion kernels)",
        },
    }


def bench_muonadamw_gpt2(steps=10, warmup=3):
    """MuonAdamW (heavyball/__init__.py:475-540) on the headline parameter set: the 49 matrices of the GPT-2-small-shaped set go
    through Muon (momentum, Newton-Schulz on the 128 x 128 tile class, the embedding's first product split along K), the 98
    vectors through Adam; one optimizer, one step counter."""
    import torch

    import heavyball_amd

    dev = torch.device("cuda:0")
    shapes = gpt2_small_shapes()
    torch.manual_seed(2)
    params = [torch.nn.Parameter(torch.randn(s, device=dev) * 0.02) for s in shapes]
    opt = heavyball_amd.MuonAdamW(params)
    grads = [torch.randn(s, device=dev) * 1e-2 for s in shapes]

    def one_step():
        for p, g in zip(params, grads):
            p.grad = g
        opt.step()

    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    flops = sum(ns5_flops(*s) for s in shapes if len(s) == 2)
    return {
        "workload": "MuonAdamW defaults, GPT-2-small-shaped 147 tensors (49 matrices through Newton-Schulz, 98 vectors through Adam), fp32",
        "ms_per_step": round(ms_step, 3),
        "ns5_algorithmic_flops_per_step": flops,
        "tflops_if_all_of_the_step_were_newton_schulz": round(flops / (ms_step * 1e-3) / 1e12, 1),
    }


def bench_reference_script(steps=300, warmup=20, windows=6):
    """The reference's own micro-benchmark (benchmarks/bench_optimizer_step.py:13, :53-81): AdamW with default arguments and
    consume_grad=False on 32 fp32 tensors of [2048, 2048] (134,217,728 elements), 20 warm-up steps, then 6 windows of 300
    steps between device synchronisations, median per-step time.  The reference's README quotes 4.15 ms for its compiled
    step on unnamed hardware; that number is shown beside ours for orientation only."""
    import statistics as st

    import torch

    import heavyball_amd

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(0)
    params = []
    for _ in range(32):
        p = torch.nn.Parameter(torch.randn((2048, 2048), device=dev, generator=gen))
        params.append(p)
    opt = heavyball_amd.AdamW(params, consume_grad=False)
    for p in params:
        p.grad = torch.randn((2048, 2048), device=dev, generator=gen)
    for _ in range(warmup):
        opt.step()
    times = []
    for _ in range(windows):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            opt.step()
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) / steps)
    ms = st.median(times) * 1e3
    n = 32 * 2048 * 2048
    return {"workload": "AdamW fp32 defaults, 32 x [2048,2048] = 134,217,728 elements, the reference's bench_optimizer_step.py protocol",
            "ms_per_step": round(ms, 4), "achieved_GBps": round(28 * n / (ms * 1e-3) / 1e9, 1), "algorithmic_bytes_per_element": 28,
            "reference_readme_ms_unknown_hardware": 4.15}  # fmt: skip


C5_SHAPES = [(2048, 2048), (2048, 8192), (8192, 2048)]
MFMA_F32_PEAK_TFLOPS = 157.3


def bench_soap_default_dim(steps=12):
    """Secondary C5 figure: the reference's default max_precond_dim = 2048 drops the 8192-wide factors, so the wide
    matrices are rotated on one side only (5.154e11 FLOP per step instead of 2.165e12)."""
    import torch

    import heavyball_amd

    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    params = [torch.nn.Parameter(torch.randn(s, device=dev) * 0.02) for s in C5_SHAPES]
    opt = heavyball_amd.SOAP(params, precondition_frequency=10, shampoo_beta=0.95)
    grad_sets = [[torch.randn(s, device=dev) * 1e-2 for s in C5_SHAPES] for _ in range(3)]
    times, refresh = [], []
    for k in range(steps + 22):  # long enough for a second basis refresh (the first one also allocates its work buffers)
        for p, g in zip(params, grad_sets[k % 3]):
            p.grad = g
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step()
        torch.cuda.synchronize()
        if k >= 2:
            (refresh if opt.param_groups[0]["is_preconditioning"] else times).append((time.perf_counter() - t0) * 1e3)
    times.sort()
    return {"max_precond_dim": 2048, "ms_per_step": round(times[len(times) // 2], 3),
            "refresh_step_ms": round(min(refresh), 3) if refresh else None, "algorithmic_flops_per_step": 515396075520}  # fmt: skip


def bench_soap_gpt2(steps=30):
    """SOAP with the default max_precond_dim on the headline parameter set: 49 matrices of 768 rows, 61 factors of 768 columns (the
    wider sides exceed max_precond_dim = 2048 and go without), 98 vectors through Adam.  The per-tensor products are mid-sized
    (108 tiles for a 768 x 2304 projection) and share launches across tensors; ``one_tensor_at_a_time`` is the same step with
    that switched off."""
    import torch

    import heavyball_amd

    dev = torch.device("cuda:0")
    shapes = gpt2_small_shapes()
    out = {"workload": "SOAP max_precond_dim 2048 (the default), precondition_frequency 10, GPT-2-small-shaped 147 tensors, fp32"}
    for key, grouped in (("ms_per_step", True), ("one_tensor_at_a_time_ms_per_step", False)):
        torch.manual_seed(5)
        params = [torch.nn.Parameter(torch.randn(s, device=dev) * 0.02) for s in shapes]
        opt = heavyball_amd.SOAP(params, precondition_frequency=10)  # as in the C5 leg: a refresh every 10th step
        opt.group_products = grouped
        grad_sets = [[torch.randn(s, device=dev) * 1e-2 for s in shapes] for _ in range(3)]
        plain, refresh = [], []
        for k in range(steps + 2):
            for p, g in zip(params, grad_sets[k % 3]):
                p.grad = g
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            opt.step()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3
            if k == 0 and grouped:
                out["init_step_ms"] = round(ms, 1)
            elif k >= 2:
                (refresh if opt.param_groups[0]["is_preconditioning"] else plain).append(ms)
        plain.sort()
        out[key] = round(plain[len(plain) // 2], 3)
        if grouped:
            out["refresh_step_ms"] = round(min(refresh), 3) if refresh else None
            if refresh:  # the reference's default refreshes the bases every second step
                out["ms_per_step_mean_at_precondition_frequency_2"] = round((out[key] + min(refresh)) / 2, 3)
        del opt, params, grad_sets
        torch.cuda.empty_cache()
    return out


def bench_soap_products(reps=3):
    """The 18 products of one SOAP step of configuration 5 on random operands, without an optimizer around them (no eigh,
    no basis refresh): a short run of a few dozen launches, meant for hardware-counter collection on the fp32 GEMM kernels.
    Prints its own JSON line."""
    import torch

    from heavyball_amd.soap import SOAP, _Gemm

    dev = torch.device("cuda:0")
    torch.manual_seed(4)
    gemm = _Gemm(dev)
    work = []
    for m, n in C5_SHAPES:
        g = torch.randn(m, n, device=dev) * 1e-2
        Q = [torch.randn(1, m, m, device=dev) / m**0.5, torch.randn(1, n, n, device=dev) / n**0.5]
        GG = [torch.zeros(1, m, m, device=dev), torch.zeros(1, n, n, device=dev)]
        work.append((g, Q, GG))

    def products():
        for g, Q, GG in work:
            SOAP._project(gemm, SOAP._project(gemm, g, Q, False), Q, True)
            SOAP._update_ggt(gemm, g, GG, 0.05, 0.95)

    products()
    stream = torch.cuda.current_stream(dev)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        products()
    e1.record(stream)
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    flops = sum(6 * (m * m * n + m * n * n) for m, n in C5_SHAPES)
    print(json.dumps({"soap_products_ms": round(ms, 3), "algorithmic_flops": flops, "achieved_TFLOPs": round(flops / ms / 1e9, 1)}))


def bench_soap(steps=30):
    """Benchmark configuration 5: SOAP (precondition_frequency 10, shampoo_beta 0.95, fp32 factors on both sides, so
    max_precond_dim 8192) on [2048,2048], [2048,8192], [8192,2048]. The first step (eigh initialisation, no update) is
    run untimed; ``steps`` further steps are timed one by one, and the median over the steps without a basis refresh is
    reported as ms_per_step, beside the time of a step with a basis refresh (every 10th) and the resulting mean.
    The roofline figure counts the 6 (m^2 n + m n^2) FLOP per matrix of the factor EMAs, projection and back-projection
    against the fp32 MFMA peak, timed with HIP events around those GEMM calls alone."""
    import torch

    import heavyball_amd
    from heavyball_amd.soap import SOAP, _Gemm

    dev = torch.device("cuda:0")
    torch.manual_seed(2)
    params = [torch.nn.Parameter(torch.randn(s, device=dev) * 0.02) for s in C5_SHAPES]
    opt = heavyball_amd.SOAP(params, precondition_frequency=10, shampoo_beta=0.95, max_precond_dim=8192)
    # six gradient sets in rotation: with one fixed gradient the 8192-wide factors would stay at rank 2048 for ever
    grad_sets = [[torch.randn(s, device=dev) * 1e-2 for s in C5_SHAPES] for _ in range(6)]
    grads = grad_sets[0]
    counter = [0]

    def one_step():
        for p, g in zip(params, grad_sets[counter[0] % len(grad_sets)]):
            p.grad = g
        counter[0] += 1
        opt.step()
        return bool(opt.param_groups[0]["is_preconditioning"])

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    one_step()
    torch.cuda.synchronize()
    init_ms = (time.perf_counter() - t0) * 1e3
    one_step()  # first real step, untimed (allocations)
    torch.cuda.synchronize()
    plain, refresh = [], []
    for _ in range(steps):
        t0 = time.perf_counter()
        fired = one_step()
        torch.cuda.synchronize()
        (refresh if fired else plain).append((time.perf_counter() - t0) * 1e3)
    plain.sort()

    # the first step of a second optimizer: what initialisation costs once the process has loaded the eigensolver
    params2 = [torch.nn.Parameter(torch.randn(s, device=dev) * 0.02) for s in C5_SHAPES]
    opt2 = heavyball_amd.SOAP(params2, precondition_frequency=10, shampoo_beta=0.95, max_precond_dim=8192)
    for p, g in zip(params2, grads):
        p.grad = g
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    opt2.step()
    torch.cuda.synchronize()
    init2_ms = (time.perf_counter() - t0) * 1e3
    del opt2, params2

    gemm = _Gemm(dev)
    stream = torch.cuda.current_stream(dev)
    work = []
    for p, g in zip(params, grads):
        st = opt.state[p][0]
        work.append((g, st["scale_by_soap_Q_3"], [m.clone() for m in st["scale_by_soap_GG_3"]]))

    def gemms():
        for g, Q, GG in work:
            back = SOAP._project(gemm, SOAP._project(gemm, g, Q, False), Q, True)
            SOAP._update_ggt(gemm, g, GG, 0.05, 0.95)
        return back

    gemms()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 3
    e0.record(stream)
    for _ in range(reps):
        gemms()
    e1.record(stream)
    torch.cuda.synchronize()
    gemm_ms = e0.elapsed_time(e1) / reps
    flops = sum(6 * (m * m * n + m * n * n) for m, n in C5_SHAPES)
    tflops = flops / (gemm_ms * 1e-3) / 1e12
    return {
        "workload": "SOAP precondition_frequency=10 shampoo_beta=0.95 max_precond_dim=8192, fp32, matrices [2048,2048] [2048,8192] [8192,2048]",
        "ms_per_step": round(plain[len(plain) // 2], 3),
        # the first refresh also pays for the allocation of its work buffers; the figures are for the ones after it
        "ms_per_step_mean_with_refresh": round((9 * plain[len(plain) // 2] + min(refresh)) / 10, 3) if refresh else None,
        "refresh_step_ms": round(min(refresh), 3) if refresh else None,
        "first_refresh_step_ms": round(refresh[0], 3) if refresh else None,
        "init_step_ms": round(init_ms, 1),
        "init_step_ms_second_optimizer": round(init2_ms, 1),
        "gemm_ms": round(gemm_ms, 3),
        "roofline": {
            "bound": "mfma",
            "achieved": round(tflops, 1),
            "peak": MFMA_F32_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(tflops / MFMA_F32_PEAK_TFLOPS, 4),
            "traffic": None,
            "algorithmic_flops_per_step": flops,
            "kernel": "hb::sgemm_big_kernel / hb::sgemm_kernel (6 products per matrix: 2 projection, 2 back-projection, 2 factor EMAs; the 8192-wide factor products compute the upper triangle and mirror it, counted at their full 2 n^2 k FLOP)",
        },
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--rounding", default="philox", choices=["philox", "half"])
    ap.add_argument("--no-muon", action="store_true", help="skip the Muon / Newton-Schulz leg (Benchmark configuration 4)")
    ap.add_argument("--no-soap", action="store_true", help="skip the SOAP leg (Benchmark configuration 5)")
    ap.add_argument("--no-8b", action="store_true", help="skip the legs on the Llama-3-8B-shaped parameter set (112 GB of device memory)")
    ap.add_argument("--soap-products", action="store_true",
                    help="run only the 18 fp32 products of one SOAP step on random operands (for hardware-counter runs) and exit")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch hb_copy_probe on 1 GiB three times (the yardstick for rocprofv3 FETCH_SIZE / WRITE_SIZE runs)")
    ap.add_argument("--kernel-launches", type=int, default=50, help="back-to-back launches for the HIP-event kernel timing")
    ap.add_argument("--windows", type=int, default=5, help="timed windows of --steps steps each; the median window is reported")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every element of the first-order step is independent, so it would shard without any exchange)", file=sys.stderr)
        sys.exit(2)

    import torch

    import heavyball_amd
    from heavyball_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(3)
    if args.soap_products:
        bench_soap_products()
        return
    first = bench_first_order(args.config, args.steps, args.warmup, args.kernel_launches, args.rounding, args.windows)
    total = first["config"]["elements"]
    out = {
        "metric": METRIC,
        "value": first["ms_per_step"],
        "unit": "ms/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": first["ms_per_step"],
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": first["config"],
        "elements_per_s": first["elements_per_s"],
        "windows": first["windows"],
        "ms_per_step_windows": first["ms_per_step_windows"],
        "host_issue_ms_per_step": first["host_issue_ms_per_step"],
        "kernel_ms": first["kernel_ms"],
        "roofline": first["roofline"],
    }
    dev = torch.device("cuda:0")
    L = _lib.lib()
    stream = torch.cuda.current_stream(dev)
    if args.calibrate:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        b = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        a.zero_()
        for _ in range(3):
            _lib.check(L.hb_copy_probe(a.data_ptr(), b.data_ptr(), 1 << 30, stream.cuda_stream))
        torch.cuda.synchronize()
        del a, b
    torch.cuda.empty_cache()
    out["adamw_reference_script"] = bench_reference_script()
    torch.cuda.empty_cache()
    if not args.no_muon:
        out["ns5"] = bench_muon()
        out["muonadamw_gpt2"] = bench_muonadamw_gpt2()
    if not args.no_soap:
        torch.cuda.empty_cache()
        out["soap"] = bench_soap()
        torch.cuda.empty_cache()
        out["soap"]["default_max_precond_dim"] = bench_soap_default_dim()
        torch.cuda.empty_cache()
        out["soap_gpt2"] = bench_soap_gpt2()
    if args.config == "c2" and not args.no_8b:
        # the 8B-shaped parameter set (benchmark configuration 3), under the headline's optimizer and under its own
        torch.cuda.empty_cache()
        free, _ = torch.cuda.mem_get_info(dev)
        if free < 200 * 2**30:
            out["llama8b"] = {"skipped": f"{free / 2**30:.0f} GiB of device memory free, the 8B-shaped set wants 200"}
        else:
            out["llama8b"] = {}
            for name in ("c2l", "c3nc", "c3"):
                leg = bench_first_order(name, 5, 2, 5, args.rounding, windows=3)
                out["llama8b"][name] = {k: leg[k] for k in ("config", "ms_per_step", "windows", "host_issue_ms_per_step", "kernel_ms",
                                                            "elements_per_s", "roofline")}  # fmt: skip
                torch.cuda.empty_cache()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.config, total)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
