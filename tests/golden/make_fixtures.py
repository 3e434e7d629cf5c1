"""Writes the golden vectors under tests/golden/ by running the reference itself.

Run once, in a container that has the reference checkout, on CPU:

    python tests/golden/make_fixtures.py [/root/reference [case names...]]

It imports optimi from that path, drives its optimizer classes with
``triton=False, foreach=False`` (the PyTorch for-loop path) on small seeded
tensors, and stores inputs (initial params, the gradient of every step) and
outputs (params and every state tensor after selected steps) as ``.npz``
files.  bf16 tensors are stored as their raw 16-bit patterns (uint16), fp16 as numpy float16.

The fixtures are data only; the tests read them with ``numpy.load`` and never
need the reference.  Each case is described in ``CASES`` below, which the tests
import to know the hyper-parameters of a fixture.
"""

from __future__ import annotations

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# tensor shapes of every case: one 2-D tensor whose size is not a multiple of any
# vector width, one small 1-D tensor
SHAPES = [(33, 37), (256,)]
SNAP_STEPS = (1, 3)  # besides the last step: lerp uses its large-weight branch at t<=2

ADAMW = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
LION = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
SADAMW = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
ADAN = dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2)
SGD = dict(lr=1e-2, momentum=0.9, weight_decay=1e-2)
RADAM = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)

# name -> (class name, kwargs, dtype, mode, n_steps)
# dtype "a+b": a parameter group of mixed dtypes - the 2-D tensor has dtype a, the 1-D tensor dtype b
# (a low-precision weight matrix and an fp32 norm weight, what optimi.utils.to_low_precision leaves behind).
# mode "group": optimizer.step() on the whole list.
# mode "release": per-tensor step(param=p) in reverse order, accumulate-only on
#                 micro-steps where (i+1) % 4 != 0 (optimizer accumulation).
# mode "functional": the functional form on explicit lists of state tensors, one shared step counter.
# mode "functional_release": the functional form on bare tensors with gradient_release=True, one
#                 counter per tensor, reverse order, the same accumulation pattern as "release".
CASES = {
    "adam_fp32_l2": ("Adam", dict(ADAMW, decouple_wd=False), "float32", "group", 10),
    "adam_fp32_nowd": ("Adam", dict(ADAMW, weight_decay=0.0), "float32", "group", 10),
    "adamw_fp32": ("AdamW", dict(ADAMW), "float32", "group", 10),
    "adamw_bf16_kahan": ("AdamW", dict(ADAMW), "bfloat16", "group", 10),
    "adamw_bf16_kahan_bigwd": ("AdamW", dict(ADAMW, lr=1e-2, weight_decay=1.0), "bfloat16", "group", 10),
    "adamw_bf16_kahan_declr": ("AdamW", dict(ADAMW, weight_decay=1e-5, decouple_lr=True), "bfloat16", "group", 10),
    "adamw_bf16_plain": ("AdamW", dict(ADAMW, kahan_sum=False), "bfloat16", "group", 10),
    "adam_bf16_kahan_l2": ("Adam", dict(ADAMW, decouple_wd=False), "bfloat16", "group", 10),
    "lion_fp32": ("Lion", dict(LION), "float32", "group", 10),
    "lion_bf16_kahan": ("Lion", dict(LION), "bfloat16", "group", 10),
    "lion_bf16_plain": ("Lion", dict(LION, kahan_sum=False), "bfloat16", "group", 10),
    "lion_bf16_kahan_declr": ("Lion", dict(LION, weight_decay=1e-2, decouple_lr=True, max_lr=3e-4), "bfloat16", "group", 10),
    "stableadamw_fp32": ("StableAdamW", dict(SADAMW), "float32", "group", 10),
    "stableadamw_bf16_kahan": ("StableAdamW", dict(SADAMW), "bfloat16", "group", 10),
    "stableadamw_bf16_plain": ("StableAdamW", dict(SADAMW, kahan_sum=False), "bfloat16", "group", 10),
    "stableadamw_bf16_kahan_declr": ("StableAdamW", dict(SADAMW, weight_decay=1e-3, decouple_lr=True, max_lr=2e-3), "bfloat16", "group", 10),
    "adan_fp32": ("Adan", dict(ADAN), "float32", "group", 10),
    "adan_bf16_kahan": ("Adan", dict(ADAN, kahan_sum=True), "bfloat16", "group", 10),
    "adan_bf16_plain": ("Adan", dict(ADAN), "bfloat16", "group", 10),
    "adan_bf16_kahan_declr": ("Adan", dict(ADAN, kahan_sum=True, decouple_lr=True, weight_decay=1e-3), "bfloat16", "group", 10),
    "adamw_fp32_release": ("AdamW", dict(ADAMW), "float32", "release", 8),
    "adamw_bf16_kahan_release": ("AdamW", dict(ADAMW), "bfloat16", "release", 8),
    "lion_bf16_kahan_release": ("Lion", dict(LION), "bfloat16", "release", 8),
    "stableadamw_bf16_kahan_release": ("StableAdamW", dict(SADAMW), "bfloat16", "release", 8),
    "adan_bf16_kahan_release": ("Adan", dict(ADAN, kahan_sum=True), "bfloat16", "release", 8),
    # with beta2 = 0.99 RAdam/Ranger take the unrectified step for t <= 5 and the rectified one from t = 6
    "sgd_fp32_l2": ("SGD", dict(SGD), "float32", "group", 10),
    "sgd_fp32_nomomentum": ("SGD", dict(SGD, momentum=0.0, decouple_wd=True), "float32", "group", 10),
    "sgd_bf16_kahan": ("SGD", dict(SGD, decouple_wd=True), "bfloat16", "group", 10),
    "sgd_bf16_kahan_dampening": ("SGD", dict(SGD, dampening=True, torch_init=True), "bfloat16", "group", 10),
    "sgd_bf16_plain_nomomentum": ("SGD", dict(SGD, momentum=0.0, kahan_sum=False), "bfloat16", "group", 10),
    "sgd_bf16_kahan_release": ("SGD", dict(SGD, decouple_wd=True), "bfloat16", "release", 8),
    "radam_fp32": ("RAdam", dict(RADAM, decouple_wd=True), "float32", "group", 10),
    "radam_bf16_kahan": ("RAdam", dict(RADAM, decouple_wd=True), "bfloat16", "group", 10),
    "radam_bf16_plain_l2": ("RAdam", dict(RADAM, kahan_sum=False), "bfloat16", "group", 10),
    "radam_bf16_kahan_release": ("RAdam", dict(RADAM, decouple_wd=True), "bfloat16", "release", 8),
    "ranger_fp32": ("Ranger", dict(RADAM), "float32", "group", 13),
    "ranger_bf16_kahan": ("Ranger", dict(RADAM), "bfloat16", "group", 13),
    "ranger_bf16_plain": ("Ranger", dict(RADAM, kahan_sum=False, k=3, alpha=0.8), "bfloat16", "group", 10),
    "ranger_bf16_kahan_release": ("Ranger", dict(RADAM, k=4), "bfloat16", "release", 8),
    # fp16: gradients of std 1e-3 square into fp16's subnormal range, which the states must round into
    "adamw_fp16_kahan": ("AdamW", dict(ADAMW), "float16", "group", 10),
    "adamw_fp16_kahan_release": ("AdamW", dict(ADAMW), "float16", "release", 8),
    "lion_fp16_kahan": ("Lion", dict(LION), "float16", "group", 10),
    "stableadamw_fp16_kahan": ("StableAdamW", dict(SADAMW), "float16", "group", 10),
    # eps 1e-8 is 0 in fp16: where exp_avg_sq underflows to 0 as well the reference divides 0 by 0,
    # and those elements are NaN from the first step on; the kernels must produce NaN in the same places
    "adan_fp16_kahan": ("Adan", dict(ADAN, kahan_sum=True), "float16", "group", 10),
    "adan_fp16_kahan_eps1e-6": ("Adan", dict(ADAN, kahan_sum=True, eps=1e-6), "float16", "group", 10),
    "sgd_fp16_kahan": ("SGD", dict(SGD, decouple_wd=True), "float16", "group", 10),
    "ranger_fp16_plain": ("Ranger", dict(RADAM, kahan_sum=False, k=3), "float16", "group", 10),
    # Adam-style decay in Adan: only the functional form takes adam_wd (the class never forwards it,
    # optimi/adan.py:181-203), so these cases drive optimi.adan(...) itself with explicit state lists
    "adan_fp32_adamwd_functional": ("Adan", dict(ADAN, adam_wd=True), "float32", "functional", 10),
    "adan_bf16_plain_adamwd_functional": ("Adan", dict(ADAN, adam_wd=True), "bfloat16", "functional", 10),
    "adan_bf16_kahan_adamwd_functional": ("Adan", dict(ADAN, adam_wd=True, kahan_sum=True), "bfloat16", "functional", 10),
    "adan_bf16_kahan_adamwd_declr_functional_release": (
        "Adan", dict(ADAN, adam_wd=True, kahan_sum=True, decouple_lr=True, weight_decay=1e-3, max_lr=2e-3),
        "bfloat16", "functional_release", 8),
    # one parameter group holding a 16-bit matrix and an fp32 vector: the group's Kahan flag comes on because of the
    # former (optimi/adam.py:100-102) and must not touch the latter
    "adamw_mixed_bf16_fp32": ("AdamW", dict(ADAMW), "bfloat16+float32", "group", 10),
    "adamw_mixed_bf16_fp32_release": ("AdamW", dict(ADAMW), "bfloat16+float32", "release", 8),
    "lion_mixed_fp16_fp32": ("Lion", dict(LION), "float16+float32", "group", 10),
    "stableadamw_mixed_bf16_fp32_declr": ("StableAdamW", dict(SADAMW, weight_decay=1e-3, decouple_lr=True, max_lr=2e-3), "bfloat16+float32", "group", 10),
    "adan_mixed_bf16_fp32_kahan": ("Adan", dict(ADAN, kahan_sum=True), "bfloat16+float32", "group", 10),
    "ranger_mixed_bf16_fp32": ("Ranger", dict(RADAM, k=3), "bfloat16+float32", "group", 10),
}

# The seed each committed fixture's inputs were drawn with.  Literal, so that adding a case can
# never move another case's inputs; tests/test_oracle_golden.py regenerates every ``in.*`` array
# from these and compares it with the stored file.
SEEDS = {
    "adam_bf16_kahan_l2": 1000, "adam_fp32_l2": 1001, "adam_fp32_nowd": 1002, "adamw_bf16_kahan": 1003,
    "adamw_bf16_kahan_bigwd": 1004, "adamw_bf16_kahan_declr": 1005, "adamw_bf16_kahan_release": 1006,
    "adamw_bf16_plain": 1007, "adamw_fp16_kahan": 1008, "adamw_fp16_kahan_release": 1009, "adamw_fp32": 1008,
    "adamw_fp32_release": 1009, "adan_bf16_kahan": 1010, "adan_bf16_kahan_declr": 1011,
    "adan_bf16_kahan_release": 1012, "adan_bf16_plain": 1013, "adan_fp16_kahan": 1016,
    "adan_fp16_kahan_eps1e-6": 1017, "adan_fp32": 1014, "lion_bf16_kahan": 1015, "lion_bf16_kahan_declr": 1016,
    "lion_bf16_kahan_release": 1017, "lion_bf16_plain": 1018, "lion_fp16_kahan": 1022, "lion_fp32": 1019,
    "radam_bf16_kahan": 99496, "radam_bf16_kahan_release": 79847, "radam_bf16_plain_l2": 54359, "radam_fp32": 40693,
    "ranger_bf16_kahan": 4133, "ranger_bf16_kahan_release": 39772, "ranger_bf16_plain": 92748,
    "ranger_fp16_plain": 71565, "ranger_fp32": 78265, "sgd_bf16_kahan": 77739, "sgd_bf16_kahan_dampening": 43561,
    "sgd_bf16_kahan_release": 79477, "sgd_bf16_plain_nomomentum": 79529, "sgd_fp16_kahan": 69834,
    "sgd_fp32_l2": 91009, "sgd_fp32_nomomentum": 57540, "stableadamw_bf16_kahan": 1020,
    "stableadamw_bf16_kahan_declr": 1021, "stableadamw_bf16_kahan_release": 1022, "stableadamw_bf16_plain": 1023,
    "stableadamw_fp16_kahan": 1028, "stableadamw_fp32": 1024,
    "adan_fp32_adamwd_functional": 3001, "adan_bf16_plain_adamwd_functional": 3002,
    "adan_bf16_kahan_adamwd_functional": 3003, "adan_bf16_kahan_adamwd_declr_functional_release": 3004,
    "adamw_mixed_bf16_fp32": 4001, "adamw_mixed_bf16_fp32_release": 4002, "lion_mixed_fp16_fp32": 4003,
    "stableadamw_mixed_bf16_fp32_declr": 4004, "adan_mixed_bf16_fp32_kahan": 4005, "ranger_mixed_bf16_fp32": 4006,
}


def case_seed(name: str) -> int:
    return SEEDS[name]


STATE_KEYS = ("exp_avg", "exp_avg_sq", "exp_avg_diff", "prev_grad", "la_param", "kahan_comp")


def to_np(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()  # float16 is stored as numpy float16, bf16 as raw uint16


def grad_scale(step: int) -> float:
    """Gradient std per step.  Varies so StableAdamW's RMS clip is above 1 on some steps."""
    return 1e-3 * (1.0, 1.0, 4.0, 0.5, 2.0)[step % 5]


def case_dtypes(dtype_name: str) -> list[torch.dtype]:
    """The dtype of every tensor of a case: "bfloat16" -> all bf16, "bfloat16+float32" -> one each."""
    names = dtype_name.split("+")
    return [getattr(torch, names[i % len(names)]) for i in range(len(SHAPES))]


def make_inputs(dtype, n_steps: int, seed: int):
    """``dtype``: one torch dtype for every tensor, or a list with one per tensor."""
    dtypes = list(dtype) if isinstance(dtype, (list, tuple)) else [dtype] * len(SHAPES)
    gen = torch.Generator().manual_seed(seed)
    params, grads = [], []
    for shape, dt in zip(SHAPES, dtypes):
        p = torch.randn(shape, generator=gen) * 0.02
        p.view(-1)[:2] = torch.tensor([0.0, 1.0])
        params.append(p.to(dt))
    for t in range(n_steps):
        gs = []
        for shape, dt in zip(SHAPES, dtypes):
            g = torch.randn(shape, generator=gen) * grad_scale(t)
            # special values: zero, below eps, large, and a sign flip partner
            g.view(-1)[:6] = torch.tensor([0.0, 1e-9, -1e-9, 1.0, -0.5, 3e-7])
            gs.append(g.to(dt))
        grads.append(gs)
    return params, grads


def snapshot(out: dict, tag: str, params, opt):
    for i, p in enumerate(params):
        out[f"{tag}.param.{i}"] = to_np(p)
        st = opt.state[p]
        for key in STATE_KEYS:
            if key in st and torch.is_tensor(st[key]) and st[key].numel() == p.numel():
                out[f"{tag}.{key}.{i}"] = to_np(st[key])


def run_case(optimi, name: str, seed: int) -> dict:
    cls_name, kwargs, dtype_name, mode, n_steps = CASES[name]
    p0, grads = make_inputs(case_dtypes(dtype_name), n_steps, seed)
    out = {}
    for i, p in enumerate(p0):
        out[f"in.param.{i}"] = to_np(p)
    for t, gs in enumerate(grads):
        for i, g in enumerate(gs):
            out[f"in.grad.{t}.{i}"] = to_np(g)

    params = [torch.nn.Parameter(p.clone()) for p in p0]
    release = mode == "release"
    opt = getattr(optimi, cls_name)(params, triton=False, foreach=False, gradient_release=release, **kwargs)
    for t in range(n_steps):
        if release:
            opt.optimizer_accumulation = (t + 1) % 4 != 0
            for i in reversed(range(len(params))):
                params[i].grad = grads[t][i].clone()
                opt.step(param=params[i])
                opt.zero_grad(param=params[i])
        else:
            for p, g in zip(params, grads[t]):
                p.grad = g.clone()
            opt.step()
            opt.zero_grad()
        if (t + 1) in SNAP_STEPS or t + 1 == n_steps:
            snapshot(out, f"out.{t + 1}", params, opt)
    return out


def run_functional_adan(optimi, name: str, seed: int) -> dict:
    """Drives the reference's functional ``adan`` (optimi/adan.py:236-350), states made as the class
    makes them (optimi/adan.py:104-120)."""
    _, kwargs, dtype_name, mode, n_steps = CASES[name]
    dtype = getattr(torch, dtype_name)
    p0, grads = make_inputs(dtype, n_steps, seed)
    out = {}
    for i, p in enumerate(p0):
        out[f"in.param.{i}"] = to_np(p)
    for t, gs in enumerate(grads):
        for i, g in enumerate(gs):
            out[f"in.grad.{t}.{i}"] = to_np(g)

    kw = dict(kwargs)
    b1, b2, b3 = kw.pop("betas")
    kahan = bool(kw.pop("kahan_sum", False)) and dtype != torch.float32
    hyper = dict(lr=kw.pop("lr"), beta1=b1, beta2=b2, beta3=b3, weight_decay=kw.pop("weight_decay"), eps=kw.pop("eps"),
                 decouple_lr=kw.pop("decouple_lr", False), max_lr=kw.pop("max_lr", None), adam_wd=kw.pop("adam_wd"),
                 kahan_sum=kahan, foreach=False, triton=False)
    assert not kw, kw
    params = [p.clone() for p in p0]
    states = [dict(exp_avg=torch.zeros_like(p), exp_avg_diff=torch.zeros_like(p), exp_avg_sq=torch.zeros_like(p),
                   prev_grad=g.clone().mul_(-1), kahan_comp=torch.zeros_like(p) if kahan else None,
                   step=torch.tensor(0, dtype=torch.int32)) for p, g in zip(params, grads[0])]
    group_step = torch.tensor(0, dtype=torch.int32)
    col = lambda key: [st[key] for st in states]  # noqa: E731

    def snap(tag):
        for i, (p, st) in enumerate(zip(params, states)):
            out[f"{tag}.param.{i}"] = to_np(p)
            for key in STATE_KEYS:
                if key in st and torch.is_tensor(st[key]):
                    out[f"{tag}.{key}.{i}"] = to_np(st[key])

    for t in range(n_steps):
        if mode == "functional_release":
            accumulate = (t + 1) % 4 != 0
            for i in reversed(range(len(params))):
                st = states[i]
                optimi.adan(params[i], grads[t][i].clone(), st["exp_avg"], st["exp_avg_diff"], st["exp_avg_sq"],
                            st["prev_grad"], st["kahan_comp"], step=st["step"], gradient_release=True,
                            optimizer_accumulation=accumulate, **hyper)
        else:
            optimi.adan(params, [g.clone() for g in grads[t]], col("exp_avg"), col("exp_avg_diff"), col("exp_avg_sq"),
                        col("prev_grad"), col("kahan_comp") if kahan else None, step=group_step, gradient_release=False,
                        optimizer_accumulation=False, **hyper)
        if (t + 1) in SNAP_STEPS or t + 1 == n_steps:
            snap(f"out.{t + 1}")
    return out


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, ref)
    import optimi  # noqa: E402  (the reference; CPU for-loop path only)

    torch.set_num_threads(1)
    only = set(sys.argv[2:])
    for name in sorted(CASES):
        if only and name not in only:
            continue
        functional = CASES[name][3].startswith("functional")
        out = (run_functional_adan if functional else run_case)(optimi, name, case_seed(name))
        path = os.path.join(HERE, f"{name}.npz")
        np.savez_compressed(path, **out)
        print(f"{name}: {len(out)} arrays, {os.path.getsize(path) / 1024:.1f} KiB")


if __name__ == "__main__":
    main()
