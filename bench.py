"""Headline benchmark: one full DistributedShampoo step on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W
        [--workload llama3_8b_layer|gpt2_small|cfg1|llama3_8b_layer_soap|large_block_eigh]

A "step" is one pass of the Shampoo hot path (factor update, batched coupled-Newton inverse
roots, grafting, preconditioning, parameter update) over one batch of synthetic gradients
that already sit in HBM.  Prints ONE JSON line with the metric, a roofline object for the
dominant kernel (the grouped fp32 MFMA GEMM of the Newton iteration, timed live with HIP
events on the stream it is launched on) and a cpu_baseline object (the CPU oracle timed on
this box's host cores: on the whole workload where that takes a minute or two, with a bounded,
scaled sample beside it as a cross-check; on a bounded sample alone where the workload amortizes
an eigendecomposition or QR refresh), next to a torch_gpu_baseline object (the same oracle's torch
ops on this GPU: what the reference's own code path costs here).  Every step draws its own
gradient set.  The default workload's line also carries "other_workloads": the other four benchmark
configurations timed natively in the same process, one amortisation period each, without baselines
(--no-other-workloads skips them).  `--gemm-standalone` times stand-alone launches of the grouped GEMM
through the C ABI instead of a workload.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # benchmark configuration 3: one Llama-3-8B decoder layer, blocks <= 2048, Newton every step
    "llama3_8b_layer": dict(
        shapes=[(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096),
                (4096, 14336), (4096,), (4096,)],
        max_preconditioner_dim=2048, grad_std=1e-2, lr=1e-3, betas=(0.9, 0.999), epsilon=1e-12,
        graft_beta2=0.999, graft_eps=1e-8,
    ),
    # benchmark configuration 2: GPT-2-small parameter set, blocks <= 1024 (ragged)
    "gpt2_small": dict(
        shapes=sum(([(2304, 768), (768, 768), (3072, 768), (768, 3072), (768,), (768,)] for _ in range(12)), [])
        + [(50257, 768)],
        max_preconditioner_dim=1024, grad_std=0.02, lr=1e-3, betas=(0.9, 0.999), epsilon=1e-12,
        graft_beta2=0.999, graft_eps=1e-8,
        # the ragged 81 x 768 tail block of the embedding gives an order-768 factor that is rank
        # deficient (and makes the reference raise) until it has seen ten gradients
        start_preconditioning_step=11, distinct_gradients=12,
    ),
    # benchmark configuration 1
    "cfg1": dict(
        shapes=[(512, 512), (512,)], max_preconditioner_dim=512, grad_std=1.0, lr=1e-3, betas=(0.9, 0.999),
        epsilon=1e-12, graft_beta2=0.999, graft_eps=1e-8,
    ),
    # benchmark configuration 4: the same Llama layer, eigenvalue-corrected Shampoo (SOAP), QR refresh every 10 steps
    "llama3_8b_layer_soap": dict(
        shapes=[(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096),
                (4096, 14336), (4096,), (4096,)],
        max_preconditioner_dim=1024, grad_std=1e-2, low_rank=(32, 1e-3), lr=1e-3, betas=(0.9, 0.999), epsilon=1e-12,
        preconditioner="soap_qr", precondition_frequency=10, start_preconditioning_step=10, grafting=None,
    ),
    # benchmark configuration 5: 4096-blocks, eigendecomposition root inverse every 50 steps
    "large_block_eigh": dict(
        shapes=[(4096, 4096)] * 8 + [(8192, 4096)] * 4,
        max_preconditioner_dim=4096, spectrum=(1e-6, 1.0), lr=1e-3, betas=(0.9, 0.999), epsilon=1e-12,
        preconditioner="eigh", precondition_frequency=50, start_preconditioning_step=50,
        graft_beta2=0.999, graft_eps=1e-8, distinct_gradients=2,
    ),
}
# HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (two
# runs, each scaled by what the counter reads for sa::copy_kernel's 1 GiB copy: 2.000 and 1.000); the
# commands and per-kernel figures are in profiles/grouped_gemm_newton_llama3_8b_layer.md.  Keyed by
# (workload, symmetric-product policy); None where no counter run was made.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {("llama3_8b_layer", 2): 9.4e9}
TRAFFIC_SOURCE = "profiles/grouped_gemm_newton_llama3_8b_layer.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, separate runs)"
DOMINANT_PHASE = {"newton": "newton_gemm", "soap_qr": "precondition_gemm", "eigh": "jacobi"}
# Deviations from the configs as literally stated, needed for the REFERENCE to run at all
# (both verified against the real reference, see tests/golden/cfg1_as_stated.json):
#  * 1-D blocks (bias / norm vectors) are left to grafting (inverse_exponent_override={1: {0: 0.0}}):
#    their rank-1 factor with epsilon=1e-12 makes the reference's Newton iteration produce
#    non-finite values and raise PreconditionerValueError at step 1.
#  * start_preconditioning_step=2: at step 1 the factor of a square Gaussian gradient block has a
#    condition number of 1e6..1e9+, below fp32 resolution; from step 2 on the EMA of two or more
#    Gram matrices is well conditioned.  Step 1 (grafting only) is part of the untimed warm-up.
START_PRECONDITIONING_STEP = 2


def build(workload: dict, device):
    import torch

    import optimizers_amd as oa

    gen = torch.Generator(device=device).manual_seed(0)
    params = [
        torch.nn.Parameter(0.02 * torch.randn(*s, device=device, generator=gen)) for s in workload["shapes"]
    ]
    kind = workload.get("preconditioner", "newton")
    if kind == "newton":
        pc = oa.RootInvShampooPreconditionerConfig(
            amortized_computation_config=oa.CoupledNewtonConfig(), inverse_exponent_override={1: {0: 0.0}})
    elif kind == "eigh":
        pc = oa.RootInvShampooPreconditionerConfig(amortized_computation_config=oa.EigenConfig())
    else:
        pc = oa.DefaultSOAPConfig
    graft = None
    if workload.get("grafting", "adam") == "adam":
        graft = oa.AdamPreconditionerConfig(beta2=workload["graft_beta2"], epsilon=workload["graft_eps"])
    opt = oa.DistributedShampoo(
        params, lr=workload["lr"], betas=workload["betas"], epsilon=workload["epsilon"],
        max_preconditioner_dim=workload["max_preconditioner_dim"],
        precondition_frequency=workload.get("precondition_frequency", 1),
        start_preconditioning_step=workload.get("start_preconditioning_step", START_PRECONDITIONING_STEP),
        preconditioner_config=pc, grafting_config=graft,
    )
    return params, opt


def make_grads(workload: dict, params, step: int, device):
    import torch

    gen = torch.Generator(device=device).manual_seed(1000 + step)
    out = []
    for p in params:
        if "spectrum" in workload and p.dim() == 2:
            # G = U diag(s) V^T with Haar U, V (QR of Gaussians) and log-uniform singular values
            lo, hi = workload["spectrum"]
            m, n = p.shape
            u, _ = torch.linalg.qr(torch.randn(m, n, device=device, generator=gen))
            w, _ = torch.linalg.qr(torch.randn(n, n, device=device, generator=gen))
            sv = torch.exp(torch.empty(n, device=device).uniform_(math.log(lo), math.log(hi), generator=gen))
            out.append(((u * sv) @ w.T).contiguous())
            continue
        g = workload.get("grad_std", 1.0) * torch.randn(p.shape, device=device, generator=gen)
        if "low_rank" in workload and p.dim() == 2:
            r, scale = workload["low_rank"]
            a = torch.randn(p.shape[0], r, device=device, generator=gen)
            c = torch.randn(r, p.shape[1], device=device, generator=gen)
            g.add_(a @ c, alpha=scale / r)
        out.append(g)
    return out


def _time_oracle(workload: dict, shapes, device, budget_s: float, timed_steps: int = 5):
    """ms/step of the oracle (the reference's algorithm as plain torch ops) on `device` for parameters of the given
    shapes, with the workload's schedule: grafting-only steps, then full steps.  Where the workload amortizes the
    root inverse / eigenbasis refresh over k > 1 steps, plain steps and steps with the amortized computation are
    timed separately (the sample alternates them) and combined for one amortized computation every k steps."""
    import torch

    from oracle.shampoo_oracle import OracleConfig, ShampooOracle

    on_gpu = device.type == "cuda"
    gen = torch.Generator(device=device).manual_seed(0)
    params = [0.02 * torch.randn(*s, device=device, generator=gen) for s in shapes]
    kind = workload.get("preconditioner", "newton")
    freq = workload.get("precondition_frequency", 1)
    sample_freq = 1 if freq == 1 else 2
    # Newton: one more grafting-only step than the native run, so that the order-2048 factor of a 1024 x 2048 block has
    # seen three gradients (rank 3072) before its first root inverse; with two its rank is exactly 2048 and whether
    # the fp32 iteration overflows depends on the draw
    start = workload.get("start_preconditioning_step", START_PRECONDITIONING_STEP) if on_gpu else START_PRECONDITIONING_STEP
    start += 1 if kind == "newton" else 0
    if sample_freq > 1:
        start = 2
    cfg = OracleConfig(
        lr=workload["lr"], betas=workload["betas"], epsilon=workload["epsilon"],
        max_preconditioner_dim=workload["max_preconditioner_dim"],
        precondition_frequency=sample_freq, start_preconditioning_step=start, preconditioner=kind,
        inverse_exponent_override={1: {0: 0.0}} if kind == "newton" else {}, grafting=workload.get("grafting", "adam"),
        grafting_beta2=workload.get("graft_beta2", 0.999), grafting_epsilon=workload.get("graft_eps", 1e-8),
    )
    opt = ShampooOracle(params, cfg)
    sample_workload = dict(workload, shapes=list(shapes))
    # gradients are drawn outside the timed region; the spectrum workload cycles through two of them like the native run
    pool = [make_grads(sample_workload, params, k, device) for k in range(2)] if "spectrum" in workload else None
    refresh, plain = [], []
    t_start = time.perf_counter()
    for step in range(1, start + 1 + timed_steps):
        grads = [g.clone() for g in pool[step % 2]] if pool else make_grads(sample_workload, params, step, device)
        if on_gpu:
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step(grads)
        if on_gpu:
            torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if step > start:  # steps after the first (cold) preconditioned one
            (refresh if step % sample_freq == 0 else plain).append(dt)
        if time.perf_counter() - t_start > budget_s and refresh and (plain or sample_freq == 1):
            break
    refresh_ms = 1e3 * sum(refresh) / len(refresh)
    plain_ms = 1e3 * sum(plain) / len(plain) if plain else refresh_ms
    ms = plain_ms + (refresh_ms - plain_ms) / freq if sample_freq > 1 else refresh_ms
    what = (f"{len(refresh)} full steps at {refresh_ms:.1f} ms/step" if sample_freq == 1 else
            f"{len(plain)} plain steps at {plain_ms:.1f} ms and {len(refresh)} steps with the amortized computation at "
            f"{refresh_ms:.1f} ms, combined for one amortized computation every {freq} steps")
    return ms, what


def torch_gpu_baseline(workload: dict, name: str, device, budget_s: float = 40.0) -> dict:
    """The reference's own code path on this GPU: the oracle's torch ops (rocBLAS GEMMs, rocSOLVER eigh / QR, a
    Python loop over blocks and factors) on device tensors, whole workload, same schedule as the CPU baseline."""
    ms, what = _time_oracle(workload, workload["shapes"], device, budget_s)
    return {"value": ms, "unit": "ms/step", "kind": "port",
            "sample": f"oracle (torch ops on {device}, fp32) on every parameter of {name}, {what}"}


def cpu_baseline(workload: dict, name: str, budget_s: float = 25.0, whole: bool = True) -> dict:
    """Times the CPU oracle (port of the reference algorithm, plain torch on the host cores).

    whole=True (Newton workloads, the default run): EVERY parameter of the workload, the native run's schedule
    (grafting-only steps, one untimed first preconditioned step, then two timed full steps): nothing is extrapolated.
    A bounded sample (the smallest 2-D parameters, scaled to the whole workload by d^3-weighted factor work) is timed
    as well and reported beside it as a cross-check; for the workloads that amortize an eigendecomposition or a QR
    refresh the sample is all that is timed."""
    import torch

    from optimizers_amd.blocking import partition_parameter

    b = workload["max_preconditioner_dim"]

    def cost(shape):
        c = 0.0
        for s in partition_parameter(0, shape, b):
            if s.order == 2:
                c += sum(float(d) ** 3 for d in s.shape)
        return c

    total = sum(cost(s) for s in workload["shapes"])
    # smallest 2-D parameter(s) first, up to ~2 * 2048^3-equivalents of factor work
    order = sorted((s for s in workload["shapes"] if len(s) == 2), key=cost)
    sample, acc = [], 0.0
    for s in order:
        if sample and acc + cost(s) > 4.5 * 2048.0**3:
            break
        sample.append(s)
        acc += cost(s)
    ms, what = _time_oracle(workload, sample, torch.device("cpu"), budget_s)
    sampled = {"value": ms * total / acc, "unit": "ms/step",
               "sample": f"parameters {sample}, {what}, scaled x{total / acc:.2f} by d^3-weighted factor work"}
    whole_ms = whole_what = None
    if whole and kind_of(workload) == "newton" and workload.get("precondition_frequency", 1) == 1:
        whole_ms, whole_what = _time_oracle(workload, workload["shapes"], torch.device("cpu"), budget_s=1e9, timed_steps=2)
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), model)
    except OSError:
        pass
    out = {
        "value": sampled["value"],
        "unit": "ms/step",
        "cores": torch.get_num_threads(),
        "host": f"{model}, os.cpu_count() = {os.cpu_count()}, torch threads = {torch.get_num_threads()}",
        "kind": "port",
        "sample": f"oracle (torch CPU fp32) on {sampled['sample']}",
        "extrapolated": True,
    }
    if whole_ms is not None:
        out.update(value=whole_ms, extrapolated=False,
                   sample=f"oracle (torch CPU fp32) on every parameter of {name}, {whole_what}; nothing extrapolated",
                   sampled_cross_check=sampled)
    return out


def measure(lib, name: str, workload: dict, steps: int, warmup: int, device, symmetric_newton: int, calibrate_copy: bool) -> dict:
    """Builds the workload, runs `warmup` untimed and `steps` timed steps and returns the JSON object of the run."""
    import torch

    from optimizers_amd import native

    start = workload.get("start_preconditioning_step", START_PRECONDITIONING_STEP)
    freq = workload.get("precondition_frequency", 1)
    params, opt = build(workload, device)
    n_params = sum(p.numel() for p in params)

    total = warmup + steps
    # one pre-generated gradient set per step (seed 1000 + step), up to 32 sets (28 GB on the Llama layer); only longer
    # runs, or the workloads that name a smaller number, cycle through them
    n_sets = min(total, workload.get("distinct_gradients", 32))
    grads = [make_grads(workload, params, s, device) for s in range(1, n_sets + 1)]
    torch.cuda.synchronize()

    def one_step(i: int) -> None:
        for p, g in zip(params, grads[i % n_sets]):
            p.grad = g
        opt.step()

    for i in range(warmup):
        one_step(i)
    torch.cuda.synchronize()
    if calibrate_copy:
        src = torch.ones(1 << 28, device=device)  # 1 GiB
        dst = torch.empty_like(src)
        native.check(lib.sa_copy_f32(src.data_ptr(), dst.data_ptr(), src.numel(), native.current_stream_ptr(device)), "sa_copy_f32")
        torch.cuda.synchronize()
        del src, dst

    # what one Newton iteration of each factor costs with the reference's full products: 2 d^3 per product,
    # 2 + (products of the square-and-multiply chain for M_p^root) products per iteration
    ng = opt._groups[0]
    full_product_flops_per_iteration = []
    for k, i in enumerate(ng.native_index):
        spec = ng.block_specs[i]
        slot = 0
        for dim in range(spec.order):
            if ng.selectors[k][dim]:
                root = int(round(ng.roots[k][slot]))
                chain = (root.bit_length() - 1) + (bin(root).count("1") - 1)
                full_product_flops_per_iteration.append(2.0 * spec.shape[dim] ** 3 * (2 + chain))
                slot += 1
    full_product_flops = 0.0

    lib.sa_set_profiling(1)
    phases = ("newton_gemm", "syrk", "precondition_gemm", "grafting", "apply", "jacobi", "qr_refresh", "eigenbasis_rotation",
              "tridiagonalize", "form_q", "tridiagonal_ql", "tridiagonal_eig")
    acc = {ph: [0.0, 0.0, 0] for ph in phases}  # ms, work, launches
    executed = 0.0
    iters = []
    t0 = time.perf_counter()
    for i in range(warmup, total):
        one_step(i)
        # phase timers are read after the step; the call synchronises on the recorded events only
        for ph in phases:
            ms = lib.sa_phase_ms(ph.encode())
            if ms >= 0:
                acc[ph][0] += ms
                acc[ph][1] += lib.sa_phase_flops(ph.encode())
                acc[ph][2] += lib.sa_phase_launches(ph.encode())
        executed += max(lib.sa_phase_executed_flops(b"newton_gemm"), 0.0)
        # forget this step's spans: a phase that the next step does not enter (an amortized computation) must not be read twice
        lib.sa_set_profiling(0)
        lib.sa_set_profiling(1)
        iters.append(list(opt._groups[0].last_newton_iterations))
        if kind_of(workload) == "newton":
            full_product_flops += sum(it * w for it, w in zip(iters[-1], full_product_flops_per_iteration))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.sa_set_profiling(0)
    ms_per_step = 1e3 * elapsed / steps

    kind = workload.get("preconditioner", "newton")
    dominant = DOMINANT_PHASE[kind]
    if kind == "eigh":  # whichever of the roofline-bound phases took longest
        dominant = max(("jacobi", "tridiagonalize", "precondition_gemm"), key=lambda ph: acc[ph][0])
    ng_ms, ng_flops, ng_launches = acc[dominant]
    hbm_bound = dominant == "tridiagonalize"
    achieved = ng_flops / (ng_ms * 1e-3) / (1e9 if hbm_bound else 1e12) if ng_ms > 0 else 0.0
    peak = PEAK_HBM_GBS if hbm_bound else PEAK_FP32_MFMA_TFLOPS
    roofline = {
        "kernel": {"newton_gemm": "grouped_gemm_kernel (coupled-Newton X*Mp, Mp^2, Mp^4, Mp^4*M)",
                   "precondition_gemm": "grouped_gemm_kernel (preconditioning products / eigenbasis rotations)",
                   "jacobi": "jacobi_cols_kernel + jacobi_rows_kernel + jacobi_pivot_kernel (block Jacobi sweeps)",
                   "tridiagonalize": "trd_symv_kernel (trailing matrix times Householder vector) + trd_column_kernel"}[dominant],
        "bound": "hbm" if hbm_bound else "mfma",
        "achieved": achieved,
        "peak": peak,
        "unit": "GB/s" if hbm_bound else "TFLOP/s",
        "frac": achieved / peak,
        # HBM bytes per launch: not measured by this run (hardware counters need rocprofv3); the figure, when there
        # is one for this workload and product policy, is copied from the committed counter profile named beside it
        "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get((name, symmetric_newton)),
        "traffic_source": (TRAFFIC_SOURCE if (name, symmetric_newton) in MEASURED_TRAFFIC_BYTES_PER_LAUNCH
                           else None),
        # `achieved` bills the algorithmic flops of the products issued (2 d^3 for a full product,
        # d^2 (d + 1) for a symmetric one); `executed_frac` adds the padding and the mirrored halves of
        # diagonal tiles, i.e. what the matrix cores really sustained.
        "symmetric_products_policy": symmetric_newton,
        # the same iterations billed as the reference's full products (2 d^3 each); above `executed_frac` because a
        # symmetric product computes only the tiles on and above the diagonal
        # NOT a utilisation: the reference's work per second (what its full GEMMs would have to sustain to match this time)
        "reference_full_gemm_billing_TFLOP/s": (full_product_flops / (ng_ms * 1e-3) / 1e12
                                                if (ng_ms > 0 and dominant == "newton_gemm") else None),
        "reference_full_gemm_billing_over_peak": (full_product_flops / (ng_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS
                                                  if (ng_ms > 0 and dominant == "newton_gemm") else None),
        "executed_TFLOP/s": executed / (ng_ms * 1e-3) / 1e12 if ng_ms > 0 else 0.0,
        "executed_frac": executed / (ng_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS if ng_ms > 0 else 0.0,
        "avg_launch_ms": ng_ms / max(ng_launches, 1),
        "flop_per_launch": ng_flops / max(ng_launches, 1),
        "launches": ng_launches,
    }
    detail = {}
    for ph in ("syrk", "precondition_gemm", "jacobi", "qr_refresh", "eigenbasis_rotation", "form_q"):
        ms, work, n = acc[ph]
        if ms > 0:
            detail[ph] = {"ms_per_step": ms / steps, "TFLOP/s": work / (ms * 1e-3) / 1e12,
                          "frac_of_fp32_mfma_peak": work / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS}
    for ph in ("tridiagonal_ql", "tridiagonal_eig"):
        if acc[ph][0] > 0:
            detail[ph] = {"ms_per_step": acc[ph][0] / steps}
    for ph in ("grafting", "apply", "tridiagonalize"):
        ms, work, n = acc[ph]
        if ms > 0:
            detail[ph] = {"ms_per_step": ms / steps, "GB/s": work / (ms * 1e-3) / 1e9,
                          "frac_of_hbm_peak": work / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS}
    detail[dominant] = dict(detail.get(dominant, {}), ms_per_step=ng_ms / steps)
    flat = [x for row in iters for x in row if x > 0]
    detail["newton_iterations_mean"] = sum(flat) / max(len(flat), 1)
    detail["newton_iterations_max"] = max(flat) if flat else 0

    out = {
        "metric": "shampoo_step_time",
        "value": ms_per_step,
        "unit": "ms/step",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": name,
            "parameters": n_params,
            "max_preconditioner_dim": workload["max_preconditioner_dim"],
            "precondition_frequency": freq,
            "start_preconditioning_step": start,
            "preconditioner": {"newton": "root inverse, coupled Newton", "eigh": "root inverse, eigendecomposition",
                               "soap_qr": "eigenvalue-corrected (SOAP), QR refresh"}[kind],
            "grafting": workload.get("grafting", "adam"),
            "inverse_exponent_override": "{1: {0: 0.0}}" if kind == "newton" else "{}",
        },
        "roofline": roofline,
        "phases": detail,
    }
    out["dominant_phase"] = dominant
    del opt, params, grads, ng
    torch.cuda.empty_cache()
    return out


def gemm_standalone(lib, device, reps: int = 100) -> dict:
    """Stand-alone launches of the grouped GEMM through the C ABI (sa_gemm_f32: full products, plain store): the Newton
    shapes of the Llama layer (108 x 2048^3) and of GPT-2 (400 x 768^3), operand layouts A as stored / A through its
    transpose, `reps` launches back to back timed with events on the launch stream (about 1.3 s per row: sustained
    clocks, not a burst); then the same launch with 1, 2, 4 ... rounds of resident workgroups (`rounds_sweep`), which
    shows what a launch costs once beside what it costs per round."""
    import torch

    from optimizers_amd import native

    rows = []
    for batch, n in ((108, 2048), (400, 768)):
        a = torch.randn(batch, n, n, device=device) * 0.01
        b = torch.randn(batch, n, n, device=device) * 0.01
        c = torch.empty(batch, n, n, device=device)
        st = native.current_stream_ptr(device)
        for layout, label in ((0, "A[m][k]"), (1, "A[k][m]")):
            call = lambda: native.check(lib.sa_gemm_f32(a.data_ptr(), b.data_ptr(), c.data_ptr(), n, n, n, n, n, n, layout, 0,
                                                        batch, n * n, n * n, n * n, st), "sa_gemm_f32")
            call()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                call()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / reps
            tf = 2.0 * n**3 * batch / (ms * 1e-3) / 1e12
            rows.append({"batch": batch, "order": n, "A": label, "ms_per_launch": ms, "TFLOP/s": tf,
                         "frac_of_fp32_mfma_peak": tf / PEAK_FP32_MFMA_TFLOPS})
        # the same launch with fewer problems: time against rounds of resident workgroups (1024 = 256 CUs x 4), which
        # separates what a launch costs once (ramp, last round) from what it costs per round
        sweep = []
        tiles_per_problem = ((n + 127) // 128) ** 2
        for part in (1, 2, 4, 8, 16, 32):
            nb = max(1, round(part * 1024 / tiles_per_problem))
            if nb > batch:
                break
            call = lambda: native.check(lib.sa_gemm_f32(a.data_ptr(), b.data_ptr(), c.data_ptr(), n, n, n, n, n, n, 1, 0,
                                                        nb, n * n, n * n, n * n, st), "sa_gemm_f32")
            call()
            torch.cuda.synchronize()
            k = max(20, int(400 / part))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(k):
                call()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / k
            rounds = nb * tiles_per_problem / 1024.0
            sweep.append({"batch": nb, "rounds": rounds, "ms_per_launch": ms, "ms_per_round": ms / rounds,
                          "frac_of_fp32_mfma_peak": 2.0 * n**3 * nb / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS})
        rows.append({"order": n, "A": "A[k][m]", "rounds_sweep": sweep})
        del a, b, c
    return {"metric": "grouped_gemm_standalone", "unit": "TFLOP/s", "launches_per_row": reps, "rows": rows}


def kind_of(workload: dict) -> str:
    return workload.get("preconditioner", "newton")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="default: 6, or one precondition_frequency period")
    ap.add_argument("--warmup", type=int, default=None, help="default: 3, or start_preconditioning_step")
    ap.add_argument("--workload", default="llama3_8b_layer", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--symmetric-newton", type=int, default=2, choices=(0, 1, 2),
                    help="coupled-Newton products: 0 = full GEMMs (the reference's arithmetic), 1 = upper triangle "
                         "mirrored, 2 (library default) = per factor, mirrored only while the factor's previous solve "
                         "converged within 14 iterations (condition number <~ 1e4)")
    ap.add_argument("--eigh-solver", type=int, default=0, choices=(0, 1, 2),
                    help="EigenConfig root inverse: 0 = by order (library default), 1 = block Jacobi, 2 = tridiagonalisation")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default run only: skip the native timing of the other four benchmark configurations")
    ap.add_argument("--gemm-standalone", action="store_true",
                    help="time stand-alone launches of the grouped GEMM (sa_gemm_f32, 108 products of order 2048 and 400 of "
                         "order 768, full products) instead of a workload")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB copy kernel (sa::copy_kernel) so that rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE readings can be scaled against a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one MI355X; --gpus must be 1 (no collectives, no sharding).")

    import torch

    from optimizers_amd import native

    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    device = torch.device("cuda:0")
    workload = WORKLOADS[args.workload]
    start = workload.get("start_preconditioning_step", START_PRECONDITIONING_STEP)
    freq = workload.get("precondition_frequency", 1)
    if args.steps is None:
        args.steps = 6 if freq == 1 else freq  # one full amortisation period
    if args.warmup is None:
        args.warmup = max(3, start + 1) if freq == 1 else start  # the first refresh is part of the warm-up
    if args.warmup < start:
        sys.exit(f"bench.py: --warmup must be >= {start} so that timed steps are full Shampoo steps.")
    lib = native.load()
    lib.sa_set_symmetric_newton(args.symmetric_newton)
    lib.sa_set_eigh_solver(args.eigh_solver)
    if args.gemm_standalone:
        print(json.dumps(gemm_standalone(lib, device)))
        return
    out = measure(lib, args.workload, workload, args.steps, args.warmup, device, args.symmetric_newton, args.calibrate_copy)
    if args.workload == "llama3_8b_layer" and not args.no_other_workloads:
        # the other four benchmark configurations, natively, one amortisation period each (no baselines)
        others = {}
        for name in ("cfg1", "gpt2_small", "llama3_8b_layer_soap", "large_block_eigh"):
            w = WORKLOADS[name]
            st, fr = w.get("start_preconditioning_step", START_PRECONDITIONING_STEP), w.get("precondition_frequency", 1)
            steps = 6 if fr == 1 else fr
            warm = max(3, st + 1) if fr == 1 else st
            m = measure(lib, name, w, steps, warm, device, args.symmetric_newton, False)
            r = m["roofline"]
            others[name] = {"ms_per_step": m["ms_per_step"], "steps": steps, "warmup": warm,
                            "dominant_phase": m["dominant_phase"], "bound": r["bound"], "achieved": r["achieved"],
                            "unit": r["unit"], "frac": r["frac"], "phases": m["phases"]}
        out["other_workloads"] = others
    out.pop("dominant_phase", None)
    if not args.no_cpu_baseline:
        out["torch_gpu_baseline"] = torch_gpu_baseline(workload, args.workload, device)
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline(workload, args.workload)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
