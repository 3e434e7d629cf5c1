"""Seeded random walks through the hyper-parameter space: both lerp branches (betas above and
below 0.5), zero and non-zero weight decay in each of its modes, decouple_lr with and without
max_lr, tiny and large eps, Kahan on and off, the three dtypes, whole-list and per-tensor
stepping with accumulate-only micro-steps.

* CPU: the C emulator against the torch for-loop restatement (each pinned by the reference's
  fixtures on the configurations those cover; here they pin each other elsewhere).
* GPU: the HIP kernels, through the C ABI, against the C emulator.
* Misaligned views (GPU): every other configuration again with parameters and gradients one or two
  elements off the 16-byte grid and sizes that are not multiples of the vector, against the emulator.
* Mixed lists: the same configurations with every other tensor in fp32 beside the 16-bit ones,
  one launch on the GPU (the ``_multi_mixed`` entry points).

Tensor sizes are multiples of 32 so that ATen's scalar remainder loop (which rounds
``add_(x, alpha=...)`` differently from its vector body in low precision) never runs.
"""

import random

import pytest
import torch

import golden_util as G
from oracle.forloop import ForLoopRun
from oracle.scalar import ScalarRun

SIZES = [32, 96, 512, 4128]
N_CONFIGS = 160


def draw_config(seed):
    rnd = random.Random(seed)
    name = rnd.choice(["adam", "adamw", "lion", "stableadamw", "adan", "sgd", "radam", "ranger"])
    dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    lr = rnd.choice([1e-4, 1e-3, 3e-3, 1e-2])
    h = dict(lr=lr)
    beta = lambda: rnd.choice([0.3, 0.45, 0.6, 0.9, 0.95, 0.99, 0.999])  # noqa: E731
    if name == "sgd":
        h.update(momentum=rnd.choice([0.0, 0.4, 0.9]), dampening=rnd.random() < 0.4, torch_init=rnd.random() < 0.3)
    elif name == "adan":
        h.update(betas=(beta(), beta(), beta()), adam_wd=rnd.random() < 0.5)
    else:
        h.update(betas=(beta(), beta()))
    if name not in ("lion", "sgd"):
        # 1e-8 is 0 in fp16 and would fill tensors with NaN; the fp16 fixtures cover that corner
        h.update(eps=rnd.choice([1e-6, 1e-5, 1e-3] if dtype == torch.float16 else [1e-8, 1e-6, 1e-3]))
    h.update(weight_decay=rnd.choice([0.0, 1e-5, 1e-2, 0.1]))
    if name in ("adam", "sgd", "radam", "ranger"):
        h.update(decouple_wd=rnd.random() < 0.5)
    if rnd.random() < 0.35:
        h.update(decouple_lr=True, weight_decay=rnd.choice([0.0, 1e-5, 1e-4]))
        if rnd.random() < 0.5:
            h.update(max_lr=lr * rnd.choice([1.0, 2.0, 10.0]))
    if name == "ranger":
        h.update(k=rnd.choice([2, 3, 5]), alpha=rnd.choice([0.5, 0.8]))
    if rnd.random() < 0.3 or name == "adan":
        h.update(kahan_sum=rnd.random() < 0.6)
    release = rnd.random() < 0.4
    return name, dtype, h, release, rnd.randrange(1 << 30)


def engine_mode(name, hyper):
    """Adan's Adam-style decay exists in the functional form only: those configurations drive the
    engines as a direct caller of the functional form would."""
    return dict(functional=True) if (name == "adan" and hyper.get("adam_wd")) else {}


def draw_tensors(dtype, seed, steps, mixed=False):
    """``mixed``: every other tensor is fp32 instead of ``dtype``."""
    gen = torch.Generator().manual_seed(seed)
    dts = [torch.float32 if (mixed and i % 2) else dtype for i in range(len(SIZES))]
    params = [(torch.randn(n, generator=gen) * 0.02).to(d) for n, d in zip(SIZES, dts)]
    grads = [[(torch.randn(n, generator=gen) * 1e-3 * (1.0, 4.0, 0.25)[t % 3]).to(d) for n, d in zip(SIZES, dts)]
             for t in range(steps)]
    return params, grads


# the whole-list configurations in a 16-bit dtype: the ones a mixed list can be made of
MIXED_SEEDS = [s for s in range(N_CONFIGS) if draw_config(s)[1] != torch.float32 and not draw_config(s)[3]]


def drive(engines, grads, release):
    for t, gs in enumerate(grads):
        for eng, put in engines:
            if release:
                eng.optimizer_accumulation = (t + 1) % 3 != 0
                for i in reversed(range(len(gs))):
                    eng.step_param(i, put(gs[i]))
            else:
                eng.step([put(g) for g in gs])


@pytest.mark.parametrize("seed", range(N_CONFIGS))
def test_emulator_matches_forloop(seed):
    name, dtype, hyper, release, data_seed = draw_config(seed)
    torch.set_num_threads(1)
    params, grads = draw_tensors(dtype, data_seed, 7)
    mode = engine_mode(name, hyper)
    sca = ScalarRun(name, [p.clone() for p in params], gradient_release=release, **mode, **hyper)
    ref = ForLoopRun(name, [p.clone() for p in params], gradient_release=release, **mode, **hyper)
    drive([(sca, torch.clone), (ref, torch.clone)], grads, release)
    what = f"seed {seed}: {name} {dtype} {hyper} release={release}"
    if dtype == torch.float32:
        G.compare_engines(sca, ref, what, exact=False)
    else:
        G.compare_engines(sca, ref, what, exact=name != "stableadamw")


@pytest.mark.parametrize("seed", MIXED_SEEDS)
def test_emulator_matches_forloop_on_mixed_lists(seed):
    name, dtype, hyper, _, data_seed = draw_config(seed)
    torch.set_num_threads(1)
    params, grads = draw_tensors(dtype, data_seed, 5, mixed=True)
    mode = engine_mode(name, hyper)
    sca = ScalarRun(name, [p.clone() for p in params], **mode, **hyper)
    ref = ForLoopRun(name, [p.clone() for p in params], **mode, **hyper)
    drive([(sca, torch.clone), (ref, torch.clone)], grads, False)
    G.compare_engines(sca, ref, f"seed {seed}: {name} {dtype}+fp32 {hyper}", exact=False)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", MIXED_SEEDS)
def test_hip_matches_emulator_on_mixed_lists(seed, hip_device):
    from hip_engine import HipRun

    name, dtype, hyper, _, data_seed = draw_config(seed)
    params, grads = draw_tensors(dtype, data_seed, 5, mixed=True)
    mode = engine_mode(name, hyper)
    hip = HipRun(name, [p.to(hip_device) for p in params], **mode, **hyper)
    sca = ScalarRun(name, [p.clone() for p in params], **mode, **hyper)
    drive([(hip, lambda g: g.to(hip_device)), (sca, torch.clone)], grads, False)
    G.compare_engines(hip, sca, f"seed {seed}: {name} {dtype}+fp32 {hyper}", exact=name != "stableadamw")


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(N_CONFIGS))
def test_hip_matches_emulator(seed, hip_device):
    from hip_engine import HipRun

    name, dtype, hyper, release, data_seed = draw_config(seed)
    params, grads = draw_tensors(dtype, data_seed, 7)
    mode = engine_mode(name, hyper)
    hip = HipRun(name, [p.to(hip_device) for p in params], gradient_release=release, **mode, **hyper)
    sca = ScalarRun(name, [p.clone() for p in params], gradient_release=release, **mode, **hyper)
    drive([(hip, lambda g: g.to(hip_device)), (sca, torch.clone)], grads, release)
    G.compare_engines(hip, sca, f"seed {seed}: {name} {dtype} {hyper} release={release}", exact=name != "stableadamw")


ODD_SIZES = [33, 97, 515, 4129, 8200, 7]


def _off_grid(t, k, device):
    """``t`` on ``device`` as a view that starts ``k`` elements into its buffer."""
    buf = torch.zeros(t.numel() + 16, dtype=t.dtype, device=device)
    view = buf[k:k + t.numel()].view(t.shape)
    view.copy_(t)
    return view


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(0, N_CONFIGS, 2))
def test_hip_matches_emulator_on_misaligned_views(seed, hip_device):
    from hip_engine import HipRun

    name, dtype, hyper, release, data_seed = draw_config(seed)
    gen = torch.Generator().manual_seed(data_seed)
    params = [(torch.randn(n, generator=gen) * 0.02).to(dtype) for n in ODD_SIZES]
    grads = [[(torch.randn(n, generator=gen) * 1e-3 * (1.0, 4.0, 0.25)[t % 3]).to(dtype) for n in ODD_SIZES] for t in range(5)]
    mode = engine_mode(name, hyper)
    hip = HipRun(name, [_off_grid(p, (i + seed) % 3, hip_device) for i, p in enumerate(params)], gradient_release=release,
                 **mode, **hyper)
    sca = ScalarRun(name, [p.clone() for p in params], gradient_release=release, **mode, **hyper)
    drive([(hip, lambda g: _off_grid(g, (seed // 2) % 2 + 1, hip_device)), (sca, torch.clone)], grads, release)
    G.compare_engines(hip, sca, f"seed {seed}: {name} {dtype} {hyper} release={release}, misaligned", exact=name != "stableadamw")
