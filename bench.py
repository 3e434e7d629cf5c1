#!/usr/bin/env python3
"""Optimizer-step throughput of the HIP backend on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

One "step" is one whole-list optimizer step (one launch of the fused kernel, three for
StableAdamW) over a synthetic parameter list that is already resident in HBM: params
N(0, 0.02) (norm weights 1.0), gradients N(0, 1e-3).  The default workload is the one the
headline metric is quoted on: bf16 AdamW with Kahan summation on a Llama-7B-shaped list
(290 tensors, 6,738,411,520 parameters).  Gradients cycle through a small pool of
independently drawn sets so that the timed region holds optimizer steps only.

Prints ONE JSON line on stdout.  ``value`` is parameters updated per second over the timed
region (wall clock around K steps, device synchronised on both sides).  ``roofline`` prices
the kernel alone: algorithmic bytes per step (each input read once, each output written
once) over the mean per-step device time between HIP events recorded on the launch stream.
``cpu_baseline`` times the PyTorch for-loop restatement (oracle/forloop.py) on this host's
cores on a bounded sample of the same list.

Two more workloads time gradient release instead (see release_bench):
``adamw_bf16_kahan_release_stress10k`` (10,000 small tensors, launch-bound) and
``adamw_bf16_kahan_release_llama7b``; ``--no-coalesce`` turns the parking of small tensors off.

Besides the headline workload the line carries ``extra``: the other benchmark configurations
(the fp32 MLP list, the Llama-1B list, Lion / StableAdamW / Adan on the Llama-7B list, and the two
gradient-release workloads), each measured the same way in the same process, as
``{workload: {ms_per_step, kernel_ms, achieved GB/s, frac}}``.  ``--no-extra`` leaves them out.
"""

from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth


def llama_shapes(hidden, inter, layers, vocab=32000, final_norm=False):
    shapes = [(vocab, hidden)]
    for _ in range(layers):
        shapes += [(hidden, hidden)] * 4 + [(inter, hidden)] * 2 + [(hidden, inter)] + [(hidden,)] * 2
    if final_norm:
        shapes.append((hidden,))
    shapes.append((vocab, hidden))
    return shapes


# name -> (optimizer class, kwargs, dtype name, shapes, algorithmic bytes per param per step)
def workloads():
    l7 = llama_shapes(4096, 11008, 32)
    l1 = llama_shapes(2048, 8192, 16, final_norm=True)
    mlp = [(1024, 4096), (4096,), (4096, 1024), (1024,)] * 2
    return {
        "adamw_bf16_kahan_llama7b": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "bfloat16", l7, 18),
        "adamw_bf16_kahan_declr_llama1b": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-5, decouple_lr=True), "bfloat16", l1, 18),
        "lion_bf16_kahan_llama7b": ("Lion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1), "bfloat16", l7, 14),
        "stableadamw_bf16_kahan_llama7b": ("StableAdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "bfloat16", l7, 22),
        "adan_bf16_kahan_llama7b": ("Adan", dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2, kahan_sum=True), "bfloat16", l7, 26),
        "adamw_fp32_mlp": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "float32", mlp, 28),
        "adamw_fp32_llama1b": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "float32", l1, 28),
        "adamw_fp16_kahan_llama7b": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "float16", l7, 18),
        # p, g, exp_avg, kahan_comp read; p, exp_avg, kahan_comp written
        "sgd_bf16_kahan_llama7b": ("SGD", dict(lr=1e-2, momentum=0.9, weight_decay=1e-2, decouple_wd=True), "bfloat16", l7, 14),
        "radam_bf16_kahan_llama7b": ("RAdam", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, decouple_wd=True), "bfloat16", l7, 18),
        # as Adam; every k-th step also reads and writes the slow weights (4 more bytes per param on that step)
        "ranger_bf16_kahan_llama7b": ("Ranger", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, k=6, alpha=0.5), "bfloat16", l7, 18),
        # the same list with the embeddings and the norm weights kept in fp32 (FP32_TENSORS): one launch over both
        # dtypes; 18 bytes per bf16 parameter, 28 per fp32 one
        "adamw_bf16_kahan_fp32_embeddings_norms_llama7b": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "bfloat16", l7, 18),
        # the same list as two parameter groups, as param_groups_weight_decay makes them: the 226 matrices decay, the 64
        # norm weights do not (TWO_GROUPS) - two launches per step, each group with its own device tables
        "adamw_bf16_kahan_decay_nodecay_llama7b": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "bfloat16", l7, 18),
        # the 10,000 small tensors of the gradient-release stress case stepped as one group (not among the default
        # extras): one launch of 0.3 ms, and a host walk over 10,000 parameters that takes several times as long
        # (host_issue_ms_per_step; the event pair around a step spans the host's time too)
        "adamw_bf16_kahan_stress10k": ("AdamW", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2), "bfloat16", stress_shapes(), 18),
    }


# workload -> which tensors of its list are fp32 instead of the workload's dtype
FP32_TENSORS = {
    "adamw_bf16_kahan_fp32_embeddings_norms_llama7b": lambda shape: len(shape) == 1 or shape[0] == 32000,
}


# workload -> which tensors of its list go into a second parameter group without weight decay
TWO_GROUPS = {
    "adamw_bf16_kahan_decay_nodecay_llama7b": lambda shape: len(shape) == 1,
}


# HBM bytes per step read off the hardware counters in a separate profiler run (rocprofv3 --pmc
# FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for the library's plain
# copy kernel over a known size).  bench.py cannot read the counters itself, so the line quotes
# the kept profile: workload -> (bytes per step, the file under profiles/ that shows them).
MEASURED_TRAFFIC = {
    "adamw_bf16_kahan_llama7b": (1.2134e11, "profiles/adamw_bf16_kahan_llama7b_hbm_traffic.txt"),
    "lion_bf16_kahan_llama7b": (9.439e10, "profiles/lion_stableadamw_adan_adamw1b_hbm_traffic.txt"),
    "stableadamw_bf16_kahan_llama7b": (1.4887e11, "profiles/lion_stableadamw_adan_adamw1b_hbm_traffic.txt"),
    "adan_bf16_kahan_llama7b": (1.7524e11, "profiles/lion_stableadamw_adan_adamw1b_hbm_traffic.txt"),
    "adamw_bf16_kahan_declr_llama1b": (2.170e10, "profiles/lion_stableadamw_adan_adamw1b_hbm_traffic.txt"),
    "adamw_bf16_kahan_fp32_embeddings_norms_llama7b": (1.23964e11, "profiles/adamw_mixed_dtype_and_fp32_lists_hbm_traffic.txt"),
    "adamw_fp32_llama1b": (3.3754e10, "profiles/adamw_mixed_dtype_and_fp32_lists_hbm_traffic.txt"),
    "adamw_fp32_mlp": (4.701e8, "profiles/adamw_mixed_dtype_and_fp32_lists_hbm_traffic.txt"),
}

# the benchmark configurations reported under "extra" next to the headline workload
EXTRA_WORKLOADS = [
    "adamw_fp32_mlp", "adamw_bf16_kahan_declr_llama1b", "lion_bf16_kahan_llama7b", "stableadamw_bf16_kahan_llama7b",
    "adan_bf16_kahan_llama7b", "adamw_bf16_kahan_fp32_embeddings_norms_llama7b", "adamw_bf16_kahan_decay_nodecay_llama7b",
    "adamw_bf16_kahan_release_llama7b",
    "adamw_bf16_kahan_release_stress10k",
    # the optimizers and dtypes beyond the benchmark configurations, so that every figure quoted anywhere is timed by
    # whoever runs this file
    "sgd_bf16_kahan_llama7b", "radam_bf16_kahan_llama7b", "ranger_bf16_kahan_llama7b", "adamw_fp16_kahan_llama7b",
    "adamw_fp32_llama1b",
]
RELEASE_WORKLOADS = ("adamw_bf16_kahan_release_stress10k", "adamw_bf16_kahan_release_llama7b")


def numel(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def make_tensors(shapes, dtype, device, seed, std, ones_for_1d=False, misalign=0):
    """``misalign`` = k > 0: every tensor is a view that starts k elements into its own buffer, i.e. off
    the 16-byte grid (what a view into a flat buffer or a gradient inside a bucket looks like)."""
    import torch

    gen = torch.Generator(device=device).manual_seed(seed)
    dtypes = dtype if isinstance(dtype, (list, tuple)) else [dtype] * len(shapes)
    out = []
    for s, dt in zip(shapes, dtypes):
        if ones_for_1d and len(s) == 1:
            t = torch.ones(s, dtype=dt, device=device)
        else:
            f = torch.empty(s, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)
            t = f.to(dt)
            del f
        if misalign:
            buf = torch.empty(t.numel() + 16, dtype=dt, device=device)
            view = buf[misalign:misalign + t.numel()].view(s)
            view.copy_(t)
            t = view
        out.append(t)
    return out


def cpu_baseline(cls_name, kwargs, dtype, shapes, budget_s=25.0):
    """Times the for-loop restatement on the host: the whole list when it is small, otherwise every
    distinct shape of the list on its own (1 warm-up, then the median of up to 5 steps), the
    list's time being the sum over shapes of time x multiplicity."""
    import torch

    from oracle.forloop import ForLoopRun

    name = cls_name.lower()
    total = sum(numel(s) for s in shapes)
    counts = {}
    for s in shapes:
        counts[s] = counts.get(s, 0) + 1
    groups = [(list(shapes), 1)] if total <= 64_000_000 else [([s], c) for s, c in counts.items()]
    list_seconds, n_steps = 0.0, 0
    t_begin = time.perf_counter()
    for sample, mult in groups:
        params = make_tensors(sample, dtype, "cpu", 1, 0.02, ones_for_1d=True)
        grads = make_tensors(sample, dtype, "cpu", 2, 1e-3)
        run = ForLoopRun(name, params, **kwargs)
        run.step([g.clone() for g in grads])  # warm-up, creates the states
        times = []
        while len(times) < 5:
            gs = [g.clone() for g in grads]  # the for-loop path uses grad as scratch
            t0 = time.perf_counter()
            run.step(gs)
            times.append(time.perf_counter() - t0)
            if len(times) >= 2 and time.perf_counter() - t_begin > budget_s * (n_steps + len(times)) / (n_steps + len(times) + 3):
                break
        list_seconds += mult * sorted(times)[len(times) // 2]
        n_steps += len(times)
        del run, params, grads
    what = ("whole list" if len(groups) == 1 else
            f"each of the {len(groups)} distinct shapes timed on its own, summed with its multiplicity")
    return {
        "value": total / list_seconds,
        "unit": "params/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{what}: {total} params, {list_seconds * 1e3:.1f} ms per step of the list, median of up to 5 steps per shape after "
                  f"1 warm-up ({n_steps} timed steps), host has {os.cpu_count()} logical CPUs",
    }


# What one step of each optimizer reads and writes, pass by pass: (arrays written in place, arrays only read).
# "p" is the parameter, "g" the gradient, the rest are state keys; the Kahan buffer exists for 16-bit tensors only.
ACCESS_MIX = {
    "AdamW": [(("p", "exp_avg", "exp_avg_sq", "kahan_comp"), ("g",))],
    "RAdam": [(("p", "exp_avg", "exp_avg_sq", "kahan_comp"), ("g",))],
    "Ranger": [(("p", "exp_avg", "exp_avg_sq", "kahan_comp"), ("g",))],
    "Lion": [(("p", "exp_avg", "kahan_comp"), ("g",))],
    "SGD": [(("p", "exp_avg", "kahan_comp"), ("g",))],
    "StableAdamW": [(("exp_avg", "exp_avg_sq"), ("g",)), (("p", "kahan_comp"), ("exp_avg", "exp_avg_sq"))],
    "Adan": [(("p", "exp_avg", "exp_avg_diff", "exp_avg_sq", "prev_grad", "kahan_comp"), ("g",))],
}


def mix_ceiling(cls_name, opt, params, grads, reps=5, granules=0):
    """The ceiling of a workload's access mix, measured on the workload's own tensors: the library's
    traffic probe (optimi_hip_stream_probe: the step's launch - same kernel, tiles, loads, stores, tables,
    throttle - with no arithmetic) over the arrays one step reads and writes.  A list that holds fp32 and
    16-bit tensors takes one probe launch per dtype.  Returns the mean seconds per step-equivalent.  The
    tensors hold meaningless bits afterwards, so this runs when the workload is done with them."""
    import torch

    from optimi_amd import cabi

    L = cabi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    launches = []  # (group, n, table, keep-alive, bytes, n_read, n_write)
    for written, read_only in ACCESS_MIX[cls_name]:
        for low in (True, False):
            idx = [i for i, p in enumerate(params) if (p.dtype != torch.float32) == low]
            if not idx:
                continue

            def array(key, i):
                if key == "p":
                    return params[i].data
                if key == "g":
                    return grads[i]
                return opt.state[params[i]][key]

            keys = [k for k in written + read_only if low or k != "kahan_comp"]
            n_write = len([k for k in written if low or k != "kahan_comp"])
            cols = [[array(k, i).data_ptr() for i in idx] for k in keys]
            for k in keys:
                assert all(array(k, i).numel() == params[i].numel() for i in idx), k
            table, keep = cabi.ptr_table(cols)
            # the probe moves whole 16-byte vectors: a tensor's last few bytes are left out (the stress list's odd sizes)
            sizes = cabi.i64_array((params[i].numel() * params[i].element_size()) & ~15 for i in idx)
            launches.append((cabi.Group(), len(idx), table, keep, sizes, len(keys), n_write))

    def once():
        for grp, n, table, _, sizes, n_read, n_write in launches:
            cabi.check(L.optimi_hip_stream_probe(grp.handle, n, table, sizes, n_read, n_write, granules, 0, stream),
                       "optimi_hip_stream_probe")

    for _ in range(2):
        once()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        once()
    stop.record()
    torch.cuda.synchronize()
    seconds = start.elapsed_time(stop) * 1e-3 / reps
    for grp, *_ in launches:
        grp.close()
    return seconds, "+".join(f"{r}r/{w}w" for _, _, _, _, _, r, w in launches)


def probe_sweep(args):
    """The library's traffic probe over the Llama-7B-shaped list (290 tensors, 13.5 GB per array, bf16
    values as the optimizers see them) for the access mixes of the optimizers, at the occupancy the
    library picks for each and at every occupancy around it: one JSON line, GB/s per (mix, granules).
    A workgroup that asks for g LDS granules leaves room for floor(128 / g) workgroups on a CU."""
    import torch

    from optimi_amd import cabi

    device = torch.device("cuda:0")
    shapes = llama_shapes(4096, 11008, 32)
    n_params = sum(numel(s) for s in shapes)
    arrays = [make_tensors(shapes, torch.bfloat16, device, 40 + a, 0.02 if a == 0 else 1e-3) for a in range(7)]
    L = cabi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    sizes = cabi.i64_array(numel(s) * 2 for s in shapes)
    grp = cabi.Group()
    mixes = [(2, 1), (3, 2), (4, 2), (4, 3), (5, 4), (6, 5), (7, 6)]
    sweep = [0, 5, 6, 7, 8, 9, 10, 11, 12, 14, 16, 18, 21]
    table_out = {}
    for n_read, n_write in mixes:
        table, keep = cabi.ptr_table([[t.data_ptr() for t in arrays[a]] for a in range(n_read)])
        row = {}
        for granules in sweep:
            def once():
                cabi.check(L.optimi_hip_stream_probe(grp.handle, len(shapes), table, sizes, n_read, n_write, granules, 0, stream),
                           "optimi_hip_stream_probe")
            for _ in range(2):
                once()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            for _ in range(args.steps):
                once()
            stop.record()
            torch.cuda.synchronize()
            ms = start.elapsed_time(stop) / args.steps
            row["library" if granules == 0 else str(granules)] = round((n_read + n_write) * 2 * n_params / ms / 1e6, 1)
        table_out[f"{n_read}r/{n_write}w"] = row
        del keep
    grp.close()
    print(json.dumps({"probe_sweep": table_out, "unit": "GB/s", "columns": "LDS granules per workgroup (library = the library's own choice)",
                      "list": "llama7b", "n_tensors": len(shapes), "bytes_per_array": 2 * n_params, "steps": args.steps}), flush=True)


def stress_shapes(n_tensors=10_000, lo=128, hi=65536, seed=6):
    """Sizes log-uniform in [lo, hi]: the many-small-tensors list of the gradient-release stress case."""
    import math

    import torch

    gen = torch.Generator().manual_seed(seed)
    u = torch.empty(n_tensors).uniform_(math.log(lo), math.log(hi), generator=gen)
    return [(int(n),) for n in torch.exp(u).long().clamp(lo, hi).tolist()]


def release_bench(workload, args, steps, warmup):
    """Gradient release: AdamW bf16 + Kahan stepped per tensor from real post-accumulate-grad hooks,
    in cycles of 3 accumulate-only backward passes and 1 full one.  An autograd function hands
    pre-made gradients to the parameters, so the backward pass launches no kernels of its own and
    what is timed is the engine's per-parameter work plus the optimizer.  A "step" is one backward
    pass over the list; the roofline figure counts 48 bytes per parameter per 4-pass cycle."""
    import torch

    import optimi_amd

    device = torch.device("cuda:0")
    shapes = stress_shapes() if workload.endswith("stress10k") else llama_shapes(4096, 11008, 32)
    n_params = sum(numel(s) for s in shapes)
    params = [torch.nn.Parameter(p) for p in make_tensors(shapes, torch.bfloat16, device, 0, 0.02, ones_for_1d=True)]
    grads = make_tensors(shapes, torch.bfloat16, device, 100, 1e-3)
    model = torch.nn.Module()
    model.ps = torch.nn.ParameterList(params)

    class Feed(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *ps):
            return ps[0].new_zeros(())

        @staticmethod
        def backward(ctx, grad_out):
            return tuple(g.view(g.shape) for g in grads)  # fresh tensor objects, so autograd adopts them as .grad

    def timed_passes(run, n):
        """Wall time of each of n backward passes, in ms (the device is idle at both ends of each)."""
        out = []
        for i in range(n):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            run(i)
            torch.cuda.synchronize()
            out.append((time.perf_counter() - t0) * 1e3)
        return out

    def median(xs):
        return sorted(xs)[len(xs) // 2]

    kwargs = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
    opt = optimi_amd.AdamW(params, gradient_release=True, **kwargs)
    if args.no_coalesce:
        opt.gradient_release_coalesce = 0
    if args.coalesce_numel is not None:
        opt.gradient_release_coalesce = args.coalesce_numel
    if args.coalesce_window is not None:
        opt._QUEUE_MAX_BYTES = args.coalesce_window
    optimi_amd.prepare_for_gradient_release(model, opt)

    def one_pass(i):
        opt.optimizer_accumulation = (i + 1) % 4 != 0
        Feed.apply(*params).backward()

    for i in range(warmup):
        one_pass(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        one_pass(warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    full = sum(1 for i in range(steps) if (warmup + i + 1) % 4 == 0)
    algo_bytes = n_params * (18.0 * full + 10.0 * (steps - full))
    achieved = algo_bytes / elapsed / 1e9
    # What the optimizer adds to a backward pass: the same passes with a hook that only frees the gradient
    # (the autograd engine's and this harness's share) in alternation with passes that step - four of the
    # one, one accumulation cycle of the other, three times over, each pass timed on its own; medians, since the
    # host's speed drifts over a run and a garbage collection now and then lands in a pass.
    empty_ms, stepping_ms = [], []
    for block in range(3):
        optimi_amd.remove_gradient_release(model)
        handles = [p.register_post_accumulate_grad_hook(lambda p: setattr(p, "grad", None)) for p in params]
        Feed.apply(*params).backward()
        empty_ms += timed_passes(lambda i: Feed.apply(*params).backward(), 4)
        for h in handles:
            h.remove()
        optimi_amd.prepare_for_gradient_release(model, opt)
        one_pass(2)
        stepping_ms += timed_passes(lambda i: one_pass(warmup + steps + i), 4)
    optimi_amd.remove_gradient_release(model)
    floor_ms = median(empty_ms)
    over_floor_us = (median(stepping_ms) - floor_ms) * 1e3 / len(shapes)
    out = {
        "metric": "gradient-release tensor-steps/s (AdamW bf16 Kahan, accumulation_steps=4)",
        "value": len(shapes) * steps / elapsed, "unit": "tensor-steps/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": elapsed / steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": workload, "optimizer": "AdamW", "n_tensors": len(shapes), "n_params": n_params,
                   "coalesce": opt.gradient_release_coalesce, "empty_hook_pass_ms": floor_ms,
                   "stepping_pass_ms_beside_it": median(stepping_ms), "us_per_tensor_over_empty_hook": over_floor_us,
                   "over_empty_hook_from": "medians of 12 passes each, in alternating blocks of 4, every pass timed on its own",
                   "hyper": {k: (list(v) if isinstance(v, tuple) else v) for k, v in kwargs.items()}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": None, "traffic_source": None,
                     "note": "wall clock over whole backward passes (hook dispatch included), launch-bound for small tensors; "
                             "a step is one backward pass, 3 of 4 accumulate-only (10 B/param), 1 of 4 full (18 B/param)"},
        "cpu_baseline": None,
    }
    del opt, params, grads, model
    return out


def list_bench(workload, args, steps, warmup):
    """One whole-list optimizer step per "step", through the optimizer class."""
    import torch

    import optimi_amd

    device = torch.device("cuda:0")
    cls_name, kwargs, dtype_name, shapes, bytes_per_param = workloads()[workload]
    dtype = getattr(torch, dtype_name)
    n_params = sum(numel(s) for s in shapes)
    is_fp32 = FP32_TENSORS.get(workload)
    dtypes = [torch.float32 if (is_fp32 and is_fp32(s)) else dtype for s in shapes]
    n_fp32 = sum(numel(s) for s, dt in zip(shapes, dtypes) if dt == torch.float32) if is_fp32 else 0
    if is_fp32:  # the average over the list: 28 bytes per fp32 parameter (four arrays read, three written)
        bytes_per_param = (bytes_per_param * (n_params - n_fp32) + 28 * n_fp32) / n_params

    misalign = getattr(args, "misalign", 0)
    params = [torch.nn.Parameter(p) for p in make_tensors(shapes, dtypes, device, 0, 0.02, ones_for_1d=True, misalign=misalign)]
    grad_sets = [make_tensors(shapes, dtypes, device, 100 + i, 1e-3, misalign=misalign) for i in range(max(1, args.grad_sets))]
    no_decay = TWO_GROUPS.get(workload)
    if no_decay:
        groups = [{"params": [p for p, s in zip(params, shapes) if not no_decay(s)]},
                  {"params": [p for p, s in zip(params, shapes) if no_decay(s)], "weight_decay": 0.0}]
        opt = getattr(optimi_amd, cls_name)(groups, **kwargs)
    else:
        opt = getattr(optimi_amd, cls_name)(params, **kwargs)

    issue = [0.0, 0]  # host seconds inside opt.step() (the walk over the list and the launch, no wait for the GPU), calls

    def one_step(i):
        for p, g in zip(params, grad_sets[i % len(grad_sets)]):
            p.grad = g
        t_in = time.perf_counter()
        opt.step()
        issue[0] += time.perf_counter() - t_in
        issue[1] += 1

    for i in range(max(warmup - 1, 0)):
        one_step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if warmup > 0:
        one_step(warmup - 1)
    torch.cuda.synchronize()
    warm_ms = (time.perf_counter() - t0) * 1e3 if warmup > 1 else float("inf")  # the last warm-up step, on its own

    # HIP events on the stream the kernels are launched on (torch's current stream is the one the
    # binding hands to the library).  A pair of events around every step gives the spread over steps;
    # each record also costs the GPU a few microseconds between kernels (measured on the 16.8 M fp32
    # list: 69.3 us per step with one pair around all steps, 76.8 us with a pair per step), so steps
    # of less than a millisecond are timed with one pair around the whole timed region instead.
    per_step_events = warm_ms >= 1.0
    n_pairs = steps if per_step_events else 1
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_pairs)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(n_pairs)]
    torch.cuda.synchronize()
    issue[0], issue[1] = 0.0, 0
    t0 = time.perf_counter()
    if per_step_events:
        for i in range(steps):
            starts[i].record()
            one_step(warmup + i)
            stops[i].record()
    else:
        starts[0].record()
        for i in range(steps):
            one_step(warmup + i)
        stops[0].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_ms = [a.elapsed_time(b) / (1 if per_step_events else steps) for a, b in zip(starts, stops)]
    mean_kernel_ms = sum(kernel_ms) / len(kernel_ms)

    if cls_name == "Ranger":  # average over the timed steps, of which every k-th is a Lookahead step
        k = kwargs["k"]
        slow = sum(1 for t in range(warmup + 1, warmup + steps + 1) if t % k == 0)
        bytes_per_param += 4.0 * slow / steps
    algo_bytes = bytes_per_param * n_params
    achieved = algo_bytes / (mean_kernel_ms * 1e-3) / 1e9
    traffic, source = MEASURED_TRAFFIC.get(workload, (None, None))
    out = {
        "metric": "optimizer-step params/sec + achieved HBM GB/s (% of peak), bf16 Kahan AdamW 6.7B",
        "value": n_params * steps / elapsed,
        "unit": "params/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": elapsed / steps * 1e3,
        "host_issue_ms_per_step": issue[0] / max(issue[1], 1) * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}[dtype],
        "data": "synthetic",
        "config": {"workload": workload, "optimizer": cls_name, "n_tensors": len(shapes), "n_params": n_params,
                   **({"n_params_fp32": n_fp32} if is_fp32 else {}), **({"misalign_elements": misalign} if misalign else {}),
                   **({"param_groups": [len(g["params"]) for g in opt.param_groups]} if no_decay else {}),
                   "hyper": {k: (list(v) if isinstance(v, tuple) else v) for k, v in kwargs.items()},
                   "grad_sets": len(grad_sets)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": source,
                     "bytes_per_param": bytes_per_param, "kernel_ms": mean_kernel_ms,
                     "kernel_ms_min": min(kernel_ms), "kernel_ms_max": max(kernel_ms),
                     "kernel_ms_p50": sorted(kernel_ms)[len(kernel_ms) // 2],
                     "kernel_ms_p90": sorted(kernel_ms)[min(len(kernel_ms) - 1, (len(kernel_ms) * 9) // 10)],
                     "kernel_ms_from": "one HIP event pair per step" if per_step_events
                     else "one HIP event pair around all timed steps (launch gaps included)"},
        "cpu_baseline": None,
    }
    if traffic is None:
        out["roofline"]["traffic_note"] = "no hardware-counter profile is kept for this workload"
    if not args.no_probe_mix:
        # same bytes, same tensors, same launch, no arithmetic: what this access mix can reach here
        seconds, mix = mix_ceiling(cls_name, opt, params, grad_sets[0])
        ceiling = algo_bytes / seconds / 1e9
        out["roofline"].update(mix_ceiling_gbps=ceiling, mix_ceiling_frac=ceiling / HBM_PEAK_GBPS, mix=mix,
                               frac_of_mix_ceiling=achieved / ceiling)
    del opt, params, grad_sets
    # the CPU baseline is timed for lists of one dtype only
    return out, (None if is_fp32 else (cls_name, kwargs, dtype, shapes))


def cold_cache_bench(args, steps=100, evict_bytes=1 << 30):
    """Benchmark configuration 1 (AdamW fp32 on the 16.8 M-parameter MLP list, 269 MB of arrays) when the
    list is NOT in the last-level cache at the start of a step, beside the back-to-back figure.  A training
    loop runs a forward and a backward pass between optimizer steps (the reference's own benchmark regenerates
    the gradients between steps, examples/benchmark.py:332-361), which sweeps this small list out of the
    256 MB cache; here torch's own copy kernel (plain cached loads and stores, like the kernels of a
    backward pass) moves `evict_bytes` (read) + `evict_bytes` (written) through the caches before every
    timed step, untimed.  Both load policies are timed under both
    conditions - four numbers, every step with its own HIP event pair on the launch stream."""
    import torch

    import optimi_amd

    device = torch.device("cuda:0")
    cls_name, kwargs, dtype_name, shapes, bytes_per_param = workloads()["adamw_fp32_mlp"]
    dtype = getattr(torch, dtype_name)
    n_params = sum(numel(s) for s in shapes)
    params = [torch.nn.Parameter(p) for p in make_tensors(shapes, dtype, device, 0, 0.02, ones_for_1d=True)]
    grad_sets = [make_tensors(shapes, dtype, device, 100 + i, 1e-3) for i in range(2)]
    opt = getattr(optimi_amd, cls_name)(params, **kwargs)
    src = torch.zeros(evict_bytes // 4, dtype=torch.float32, device=device)
    dst = torch.empty(evict_bytes // 4, dtype=torch.float32, device=device)

    def one_step(i):
        for p, g in zip(params, grad_sets[i % 2]):
            p.grad = g
        opt.step()

    def evict():
        dst.copy_(src)

    out = {"evict_bytes_read_and_written": 2 * evict_bytes, "steps": steps, "n_params": n_params,
           "timed": "one HIP event pair per step; the evicting copy runs before the first event"}
    for policy, resident in (("cached_loads", True), ("streaming_loads", False)):
        opt.resident_lists = resident
        for condition in ("back_to_back", "cold"):
            for i in range(5):
                one_step(i)
            starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
            stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
            torch.cuda.synchronize()
            for i in range(steps):
                if condition == "cold":
                    evict()
                starts[i].record()
                one_step(i)
                stops[i].record()
            torch.cuda.synchronize()
            us = sorted(a.elapsed_time(b) * 1e3 for a, b in zip(starts, stops))
            mean = sum(us) / len(us)
            out[f"{policy}_{condition}"] = {"kernel_us": mean, "kernel_us_p50": us[len(us) // 2],
                                            "achieved_gbps": bytes_per_param * n_params / mean / 1e3,
                                            "frac": bytes_per_param * n_params / mean / 1e3 / HBM_PEAK_GBPS}
    opt.resident_lists = False
    out["default"] = "streaming_loads (cached loads are opt-in: OptimiOptimizer.resident_lists / OPTIMI_RESIDENT)"
    del opt, params, grad_sets, src, dst
    return out


def run_workload(workload, args, steps, warmup):
    if workload in RELEASE_WORKLOADS:
        return release_bench(workload, args, steps, warmup), None
    return list_bench(workload, args, steps, warmup)


def brief(line):
    """The part of a workload's line that goes under "extra"."""
    r = line["roofline"]
    out = {"ms_per_step": line["ms_per_step"], "achieved_gbps": r["achieved"], "frac": r["frac"], "steps": line["steps"],
           "unit": line["unit"], "value": line["value"]}
    if "kernel_ms" in r:
        out.update(kernel_ms=r["kernel_ms"], kernel_ms_min=r["kernel_ms_min"], bytes_per_param=r["bytes_per_param"],
                   host_issue_ms_per_step=line["host_issue_ms_per_step"])
        if "mix_ceiling_gbps" in r:
            out.update(mix_ceiling_gbps=r["mix_ceiling_gbps"], mix=r["mix"], frac_of_mix_ceiling=r["frac_of_mix_ceiling"])
    else:
        out.update(timed="wall clock over backward passes", empty_hook_pass_ms=line["config"]["empty_hook_pass_ms"],
                   us_per_tensor_over_empty_hook=line["config"]["us_per_tensor_over_empty_hook"])
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="adamw_bf16_kahan_llama7b")
    ap.add_argument("--grad-sets", type=int, default=2)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="measure the named workload only, not the other configurations")
    ap.add_argument("--misalign", type=int, default=0,
                    help="list workloads: make every parameter and gradient a view that starts this many elements into "
                         "its buffer (off the 16-byte grid); the optimizer states stay aligned")
    ap.add_argument("--no-probe-mix", action="store_true",
                    help="list workloads: do not measure the ceiling of the workload's access mix with the library's "
                         "traffic probe after the timed steps")
    ap.add_argument("--probe-sweep", action="store_true",
                    help="instead of a workload: the traffic probe over the Llama-7B-shaped list for every optimizer's "
                         "access mix, at the library's occupancy and at every occupancy around it (--steps launches each)")
    ap.add_argument("--no-coalesce", action="store_true",
                    help="gradient-release workloads: launch every tensor from its own hook instead of parking small ones")
    ap.add_argument("--copy-probe-bytes", type=int, default=0,
                    help="also run the library's plain copy kernel over this many bytes (3 launches) before the "
                         "workload; a profiler run uses it to scale its byte counters against a known size")
    ap.add_argument("--coalesce-numel", type=int, default=None,
                    help="gradient-release workloads: park tensors of at most this many elements (default: the optimizer's)")
    ap.add_argument("--coalesce-window", type=int, default=None,
                    help="gradient-release workloads: launch when this many bytes of gradients are parked (default: the optimizer's)")
    args = ap.parse_args()

    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); the step needs no exchange between "
                 "GPUs, so a multi-GPU figure would be N independent copies of this run")

    import torch

    import optimi_amd  # noqa: F401  (fails loudly here when the HIP extension is missing)

    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device visible")
    device = torch.device("cuda:0")
    if args.copy_probe_bytes:
        from optimi_amd import cabi

        n = args.copy_probe_bytes // 16 * 16
        src = torch.zeros(n, dtype=torch.uint8, device=device)
        dst = torch.ones(n, dtype=torch.uint8, device=device)
        for _ in range(3):
            cabi.check(cabi.lib().optimi_hip_copy_probe(dst.data_ptr(), src.data_ptr(), n, torch.cuda.current_stream().cuda_stream),
                       "optimi_hip_copy_probe")
        torch.cuda.synchronize()
        del src, dst

    if args.probe_sweep:
        probe_sweep(args)
        return
    if args.workload == "adamw_fp32_mlp_cold":
        print(json.dumps({"adamw_fp32_mlp_cold": cold_cache_bench(args, steps=args.steps)}), flush=True)
        return

    # Between workloads the freed tensors stay in torch's caching allocator and are handed out again
    # (the 7B-shaped workloads share their shapes).  Returning them to the driver and allocating
    # afresh costs the later workloads 2-4 % of bandwidth on this system (AdamW on the 7B list: 18.4 ms
    # first, 18.85-18.95 ms after such a round trip; 18.4-18.5 ms when the blocks are reused), and seconds.
    out, spec = run_workload(args.workload, args, args.steps, args.warmup)
    gc.collect()
    if not args.no_extra:
        extra = {}
        for name in EXTRA_WORKLOADS:
            if name == args.workload:
                continue
            # short launches are timed over more steps: a 0.1 ms step needs many to average the host's jitter out
            steps = 200 if name == "adamw_fp32_mlp" else (40 if "llama1b" in name else (16 if name in RELEASE_WORKLOADS else 12))
            line, extra_spec = run_workload(name, args, steps, 8 if name in RELEASE_WORKLOADS else 5)
            extra[name] = brief(line)
            if name == "adamw_fp32_mlp" and extra_spec is not None and not args.no_cpu_baseline:
                # benchmark configuration 1 is the reference's own CPU-runnable case: the whole list, a few seconds
                extra[name]["cpu_baseline"] = cpu_baseline(*extra_spec, budget_s=6.0)
            gc.collect()
        extra["adamw_fp32_mlp_cold"] = cold_cache_bench(args)
        gc.collect()
        out["extra"] = extra
    if spec is not None and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(*spec)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
