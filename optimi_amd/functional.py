"""Functional optimizer steps: ``adam``, ``adamw``, ``lion``, ``stableadamw``, ``adan``, ``sgd``,
``radam``, ``ranger``.

Same keyword signatures as the reference's functional forms (optimi/adam.py:213-234,
adamw.py:78-98, lion.py:187-204, stableadamw.py:277-299, adan.py:236-260, sgd.py:213-231,
radam.py:214-235, ranger.py:230-254).  Each forms the
step scalars in Python doubles exactly where the reference does, then hands the tensors
to the HIP backend: one launch for a list, the per-tensor entry point when
``gradient_release=True``.  ``triton=True`` selects that backend; it is the only one in
this package: the deprecated ``foreach=True`` is served by the same kernels, and ``triton=False``
without it (the PyTorch for-loop path) raises instead of running a slower path behind the
caller's back.
"""

from __future__ import annotations

import math
from collections import defaultdict

import torch
from torch import Tensor

from . import backend
from .utils import debias, debias_beta

__all__ = ["adam", "adamw", "lion", "stableadamw", "adan", "sgd", "radam", "ranger"]

_LOW_PRECISION = (torch.float16, torch.bfloat16)


def _require_hip_backend(triton, foreach, gradient_release):
    """Both of the reference's accelerated selectors, ``triton=True`` and the deprecated
    ``foreach=True``, are served by the HIP kernels; the PyTorch for-loop path (both False) does
    not exist here.  foreach with gradient release is an error, as in optimi/adam.py:281-282."""
    if foreach and gradient_release:
        raise ValueError(f"Gradient release {gradient_release=} and foreach {foreach=} cannot be used together")
    if not triton and not foreach:
        raise ValueError(
            "optimi_amd implements only the fused HIP backend, selected with triton=True (or foreach=True); "
            "the PyTorch for-loop path is not part of this package"
        )


def _tick(step: Tensor) -> int:
    step.add_(1)
    return int(step.item())


def _flags(ext, *, kahan_sum, update_parameters, **more) -> int:
    f = (ext.KAHAN if kahan_sum else 0) | (ext.UPDATE if update_parameters else 0)
    for name, on in more.items():
        if on:
            f |= getattr(ext, name)
    return f


def _as_lists(*cols):
    """Accepts the reference's two calling forms: lists, or bare tensors in gradient-release mode."""
    return [[c] if (isinstance(c, Tensor) or c is None) else list(c) for c in cols]


def _buckets(params: list[Tensor]):
    """Indices of ``params`` grouped into launches: one per device, float32 tensors together with the
    tensors of one 16-bit dtype.  Keys are (device, that 16-bit dtype or float32); a device that
    holds bfloat16 and float16 parameters gets a launch for each, the float32 ones riding with
    whichever 16-bit dtype comes first."""
    low = {}
    for p in params:
        backend.check_supported(p)
        if p.dtype != torch.float32:
            low.setdefault(p.device, p.dtype)
    out = defaultdict(list)
    for i, p in enumerate(params):
        dtype = low.get(p.device, torch.float32) if p.dtype == torch.float32 else p.dtype
        out[(p.device, dtype)].append(i)
    return out


def _pick(col, idxs):
    return [col[i] for i in idxs]


def _grads_like(params, grads):
    out = []
    for p, g in zip(params, grads):
        if g.dtype != p.dtype:
            raise TypeError(f"optimi_amd: gradient dtype {g.dtype} differs from parameter dtype {p.dtype}")
        if g.is_sparse:
            raise RuntimeError("optimi_amd does not support sparse gradients")
        out.append(backend.like_param(p, g))
    return out


def _check_state(param: Tensor, state: Tensor, name: str):
    if state.device != param.device or state.dtype != param.dtype or state.numel() != param.numel() \
            or state.stride() != param.stride():
        raise RuntimeError(f"optimi_amd: {name} must have the parameter's device, dtype, size and strides "
                           f"(got {state.dtype} {tuple(state.shape)} on {state.device})")


def _validated(params, grads, states, kahan_comps, optional=()):
    """The two calling forms (lists, or bare tensors in gradient-release mode) as lists, with every
    check that can reject the call done here - before the step counter moves or a kernel runs.
    ``states`` are the per-parameter state columns; a column named in ``optional`` may hold None or
    one-element placeholders."""
    n = 1 if isinstance(params, Tensor) else len(params)
    if kahan_comps is None:
        kahan_comps = [None] * n
    cols = _as_lists(params, grads, *states, kahan_comps)
    params = cols[0]
    for c in cols[1:]:
        if len(c) != len(params):
            raise ValueError(f"optimi_amd: got {len(params)} parameters but a list of {len(c)} gradients or states")
    for p in params:
        backend.check_supported(p)
    cols[1] = _grads_like(params, cols[1])
    for j, col in enumerate(cols[2:-1]):
        for p, st in zip(params, col):
            if j in optional and _real_kahan(p, st) is None:
                continue
            _check_state(p, st, "a state tensor")
    for p, k in zip(params, cols[-1]):
        if _real_kahan(p, k) is not None:
            _check_state(p, k, "kahan_comp")
    return cols


# --------------------------------------------------------------------------------------
# Adam / AdamW
# --------------------------------------------------------------------------------------
def adam(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor],
    exp_avg_sqs: list[Tensor],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    weight_decay: float,
    eps: float,
    step: Tensor,
    decouple_wd: bool,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply an Adam or AdamW optimization step (optimi/adam.py:213-309).

    Args mirror the reference: tensors (or lists of tensors) to update, their gradients and
    states, the raw hyper-parameters, and the int32 CPU ``step`` counter, which is advanced
    here.  ``_groups`` is an optional dict the caller owns in which launch workspaces are kept;
    ``_resident`` says that the list was stepped a moment ago and is still in the GPU's last-level cache.
    """
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    params, grads, exp_avgs, exp_avg_sqs, kahan_comps = _validated(params, grads, (exp_avgs, exp_avg_sqs), kahan_comps)

    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    if weight_decay != 0:
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident,
                   DECOUPLE_WD=decouple_wd or decouple_lr)
    scalars = (lr, 1 - beta1_hat, beta2_hat, 1 - beta2_hat, weight_decay, eps, flags)

    if gradient_release:
        for p, g, m, v, k in zip(params, grads, exp_avgs, exp_avg_sqs, kahan_comps):
            ext.adam_single(p, g, m, v, _real_kahan(p, k), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "adam")
        ext.adam_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(exp_avgs, idxs), _pick(exp_avg_sqs, idxs),
                       [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


def adamw(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor],
    exp_avg_sqs: list[Tensor],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    weight_decay: float,
    eps: float,
    step: Tensor,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply an AdamW optimization step: ``adam`` with decoupled weight decay
    (optimi/adamw.py:78-143)."""
    adam(params, grads, exp_avgs, exp_avg_sqs, kahan_comps, lr=lr, beta1=beta1, beta2=beta2, weight_decay=weight_decay,
         eps=eps, step=step, decouple_wd=True, decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum,
         foreach=foreach, triton=triton, gradient_release=gradient_release,
         optimizer_accumulation=optimizer_accumulation, _groups=_groups, _resident=_resident)


# --------------------------------------------------------------------------------------
# Lion
# --------------------------------------------------------------------------------------
def lion(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor | None],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    weight_decay: float,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply a Lion optimization step (optimi/lion.py:187-266)."""
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    params, grads, exp_avgs, kahan_comps = _validated(params, grads, (exp_avgs,), kahan_comps)

    if weight_decay != 0:
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        else:
            weight_decay = 1 - lr * weight_decay
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident)
    scalars = (lr, 1 - beta1, 1 - beta2, weight_decay, flags)

    if gradient_release:
        for p, g, m, k in zip(params, grads, exp_avgs, kahan_comps):
            ext.lion_single(p, g, m, _real_kahan(p, k), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "lion")
        ext.lion_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(exp_avgs, idxs),
                       [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


# --------------------------------------------------------------------------------------
# StableAdamW
# --------------------------------------------------------------------------------------
def stableadamw(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor],
    exp_avg_sqs: list[Tensor],
    eps_sqs: list[Tensor],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    weight_decay: float,
    eps: float,
    step: Tensor,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    mean_squares: list[Tensor] | None = None,
    _groups=None,
    _resident=False,
):
    """Functional API to apply a StableAdamW optimization step (optimi/stableadamw.py:277-371).

    ``eps_sqs`` and ``mean_squares`` are accepted for signature and state-dict compatibility.
    The kernels take eps**2 rounded to the parameter dtype from ``eps`` itself (the value the
    reference stores in ``eps_sq``) and keep the RMS reduction in their own workspace, so
    neither list is read or written.
    """
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    params, grads, exp_avgs, exp_avg_sqs, kahan_comps = _validated(params, grads, (exp_avgs, exp_avg_sqs), kahan_comps)
    if decouple_lr and weight_decay != 0 and not (max_lr is not None and max_lr > 0):
        raise ValueError(f"optimi_amd: decouple_lr needs a positive max_lr, got {max_lr=}")

    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident, DECOUPLE_LR=decouple_lr)
    scalars = (lr, 1 - beta1_hat, beta2_hat, 1 - beta2_hat, weight_decay, eps,
               float(max_lr) if (decouple_lr and max_lr is not None) else 0.0, flags)

    if gradient_release:
        for p, g, m, v, k in zip(params, grads, exp_avgs, exp_avg_sqs, kahan_comps):
            grp = _workspace(_groups, p.device, p.dtype, "stableadamw_single")
            ext.stableadamw_single(grp, p, g, m, v, _real_kahan(p, k), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "stableadamw")
        ext.stableadamw_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(exp_avgs, idxs),
                              _pick(exp_avg_sqs, idxs), [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


# --------------------------------------------------------------------------------------
# Adan
# --------------------------------------------------------------------------------------
def adan(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor],
    exp_avg_diffs: list[Tensor],
    exp_avg_sqs: list[Tensor],
    prev_grads: list[Tensor],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    beta3: float,
    weight_decay: float,
    eps: float,
    step: Tensor,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    adam_wd: bool = False,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply an Adan optimization step (optimi/adan.py:236-350)."""
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    params, grads, exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads, kahan_comps = _validated(
        params, grads, (exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads), kahan_comps)

    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    beta3_hat = debias_beta(beta3, t)
    if weight_decay != 0:
        weight_decay = (lr / max_lr) * weight_decay if decouple_lr else lr * weight_decay
        weight_decay = 1 - weight_decay if adam_wd else 1 + weight_decay
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident, ADAM_WD=adam_wd)
    scalars = (lr, 1 - beta1_hat, beta2, 1 - beta2_hat, beta3_hat, 1 - beta3_hat, eps, weight_decay, flags)

    if gradient_release:
        for p, g, m, df, n, pg, k in zip(params, grads, exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads, kahan_comps):
            ext.adan_single(p, g, m, df, n, pg, _real_kahan(p, k), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "adan")
        ext.adan_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(exp_avgs, idxs), _pick(exp_avg_diffs, idxs),
                       _pick(exp_avg_sqs, idxs), _pick(prev_grads, idxs),
                       [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


# --------------------------------------------------------------------------------------
# SGD
# --------------------------------------------------------------------------------------
def sgd(
    params: list[Tensor] | Tensor,
    grads: list[Tensor] | Tensor,
    exp_avgs: list[Tensor | None] | Tensor | None,
    kahan_comps: list[Tensor | None] | Tensor | None = None,
    *,
    lr: float,
    momentum: float,
    weight_decay: float,
    dampening: bool,
    decouple_wd: bool,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply a SGD or SGDW optimization step (optimi/sgd.py:213-298)."""
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    if exp_avgs is None:
        exp_avgs = [None] * (1 if isinstance(params, Tensor) else len(params))
    # without momentum the buffer may be None or a one-element placeholder: never validated, never passed
    params, grads, exp_avgs, kahan_comps = _validated(params, grads, (exp_avgs,), kahan_comps,
                                                      optional=(0,) if momentum == 0 else ())

    if weight_decay != 0:
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident,
                   DECOUPLE_WD=decouple_wd or decouple_lr, DAMPENING=dampening)
    scalars = (lr, momentum, weight_decay, flags)

    # without momentum the buffer is None or a one-element placeholder (optimi/sgd.py:103-106)
    moms = [_real_kahan(p, m) if momentum != 0 else None for p, m in zip(params, exp_avgs)]

    if gradient_release:
        for p, g, m, k in zip(params, grads, moms, kahan_comps):
            ext.sgd_single(p, g, m, _real_kahan(p, k), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "sgd")
        ext.sgd_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(moms, idxs),
                      [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


# --------------------------------------------------------------------------------------
# RAdam and Ranger
# --------------------------------------------------------------------------------------
def _rectification(beta2: float, step: int) -> float | None:
    """Variance rectification term once the approximated SMA is longer than 5, else None
    (optimi/radam.py:269-277)."""
    rho_inf = 2 / (1 - beta2) - 1
    rho = rho_inf - 2 * step * (beta2**step) / debias(beta2, step)
    if rho > 5:
        return math.sqrt(((rho - 4) * (rho - 2) * rho_inf) / ((rho_inf - 4) * (rho_inf - 2) * rho))
    return None


def radam(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor],
    exp_avg_sqs: list[Tensor],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    weight_decay: float,
    eps: float,
    step: Tensor,
    decouple_wd: bool,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply an RAdam optimization step (optimi/radam.py:214-322)."""
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    params, grads, exp_avgs, exp_avg_sqs, kahan_comps = _validated(params, grads, (exp_avgs, exp_avg_sqs), kahan_comps)

    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    rect = _rectification(beta2, t)
    if weight_decay != 0:
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident,
                   DECOUPLE_WD=decouple_wd or decouple_lr, RECTIFY=rect is not None)
    scalars = (lr, 1 - beta1_hat, beta2_hat, 1 - beta2_hat, weight_decay, eps, rect if rect is not None else 0.0, flags)

    if gradient_release:
        for p, g, m, v, k in zip(params, grads, exp_avgs, exp_avg_sqs, kahan_comps):
            ext.radam_single(p, g, m, v, _real_kahan(p, k), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "radam")
        ext.radam_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(exp_avgs, idxs), _pick(exp_avg_sqs, idxs),
                        [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


def ranger(
    params: list[Tensor],
    grads: list[Tensor],
    exp_avgs: list[Tensor],
    exp_avg_sqs: list[Tensor],
    la_params: list[Tensor],
    kahan_comps: list[Tensor | None] | None = None,
    *,
    lr: float,
    beta1: float,
    beta2: float,
    weight_decay: float,
    eps: float,
    k: int,
    alpha: float,
    step: Tensor,
    decouple_wd: bool,
    decouple_lr: bool = False,
    max_lr: float | None = None,
    kahan_sum: bool = False,
    foreach: bool = False,
    triton: bool = False,
    gradient_release: bool = False,
    optimizer_accumulation: bool = False,
    _groups=None,
    _resident=False,
):
    """Functional API to apply a Ranger optimization step: RAdam plus Lookahead every ``k`` steps
    (optimi/ranger.py:230-344)."""
    _require_hip_backend(triton, foreach, gradient_release)
    ext = backend.ext()
    params, grads, exp_avgs, exp_avg_sqs, la_params, kahan_comps = _validated(
        params, grads, (exp_avgs, exp_avg_sqs, la_params), kahan_comps)

    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    rect = _rectification(beta2, t)
    if weight_decay != 0:
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    flags = _flags(ext, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation, RESIDENT=_resident,
                   DECOUPLE_WD=decouple_wd or decouple_lr, RECTIFY=rect is not None, LOOKAHEAD=t % k == 0)
    scalars = (lr, 1 - beta1_hat, beta2_hat, 1 - beta2_hat, weight_decay, eps, rect if rect is not None else 0.0, alpha, flags)

    if gradient_release:
        for p, g, m, v, la, kc in zip(params, grads, exp_avgs, exp_avg_sqs, la_params, kahan_comps):
            ext.ranger_single(p, g, m, v, la, _real_kahan(p, kc), *scalars)
        return
    for (device, dtype), idxs in _buckets(params).items():
        grp = _workspace(_groups, device, dtype, "ranger")
        ext.ranger_multi(grp, _pick(params, idxs), _pick(grads, idxs), _pick(exp_avgs, idxs), _pick(exp_avg_sqs, idxs),
                         _pick(la_params, idxs), [_real_kahan(params[i], kahan_comps[i]) for i in idxs], *scalars)


# --------------------------------------------------------------------------------------
def _real_kahan(param: Tensor, kahan: Tensor | None) -> Tensor | None:
    """The Kahan buffer if it is one; the 1-element placeholders the reference keeps in state
    for Triton (optimi/adam.py:103-104, lion.py:96-97) and None count as absent."""
    if kahan is None or kahan.numel() != param.numel() or kahan.dtype != param.dtype:
        return None
    return kahan


def _workspace(groups, device, dtype, tag):
    if groups is None:
        return backend.default_group(device, dtype, tag)
    key = (device.type, device.index, dtype, tag)
    grp = groups.get(key)
    if grp is None:
        with torch.cuda.device(device):
            grp = backend.ext().Group()
        groups[key] = grp
    return grp
