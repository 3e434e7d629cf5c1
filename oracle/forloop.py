"""Op-for-op CPU restatement of optimi's PyTorch for-loop optimizer step.

TEST INFRASTRUCTURE ONLY – see ``oracle/__init__.py``.

Every function issues the same in-place ATen ops, in the same order, as the
reference function it cites, so each intermediate is rounded to the tensor
dtype where the reference rounds it.  Scalars stay Python doubles until an op
narrows them, as in the reference.  Like the reference, these functions use
``grad`` as scratch: callers that need the gradient afterwards pass a clone.

Pinning status (what independently checks each function):

=========================  ====================================================
function                   pinned by
=========================  ====================================================
``debias_beta``            closed form beta*(1-beta^(t-1))/(1-beta^t); golden
                           fixtures (every optimizer run depends on it)
``adam_tensor``            golden fixtures written by the reference itself
                           (tests/golden); torch.optim.Adam/AdamW equivalence in
                           fp32; t=1 closed form; scalar C emulator bit-equality
``lion_tensor``            golden fixtures; |dp| = lr closed form at wd=0;
                           scalar C emulator bit-equality
``stableadamw_tensor``     golden fixtures; rms<=1 reduces to ``adam_tensor``;
                           scalar C emulator
``adan_tensor``            golden fixtures (class path, and the functional form with
                           ``adam_wd=True``); t=1 closed form; float64 textbook Adan in
                           both decay styles; scalar C emulator
``sgd_tensor``             golden fixtures; torch.optim.SGD equivalence in fp32;
                           scalar C emulator
``radam_tensor``           golden fixtures; torch.optim.RAdam equivalence in fp32;
                           scalar C emulator
``ranger_tensor``          golden fixtures; float64 Lookahead-over-RAdam
                           restatement; scalar C emulator
functional ``adam`` …      golden fixtures (class API and gradient-release /
                           accumulation runs of the reference)
``ForLoopRun`` on a group  golden fixtures of one parameter group holding a
of mixed dtypes            16-bit and an fp32 tensor (``*_mixed_*``)
=========================  ====================================================
"""

from __future__ import annotations

import math

import torch
from torch import Tensor

LOW_PRECISION = (torch.float16, torch.bfloat16)


# ----------------------------------------------------------------------------
# scalar prologues
# ----------------------------------------------------------------------------
def debias_beta(beta: float, step: int) -> float:
    """Debiased beta, ``(beta^t - beta) / (beta^t - 1)``  (optimi/utils.py:31-36)."""
    bt = beta**step
    return (bt - beta) / (bt - 1)


def _tick(step: Tensor) -> int:
    """Advance the int32 CPU step counter in place and read it (optimi/adam.py:261-262)."""
    step.add_(1)
    return int(step.item())


def _as_list(x):
    return [x] if isinstance(x, Tensor) or x is None else list(x)


# ----------------------------------------------------------------------------
# shared tail: p += update via Kahan buffer, or directly
# ----------------------------------------------------------------------------
def _kahan_commit(param: Tensor, grad: Tensor, kahan_comp: Tensor):
    """param += kahan_comp; kahan_comp += (old param - new param), ``grad`` is the
    scratch that holds the old param  (optimi/adam.py:388-393, lion.py:327-335,
    stableadamw.py:463-469, adan.py:452-458)."""
    grad.copy_(param.detach())
    param.add_(kahan_comp)
    kahan_comp.add_(grad.sub_(param))


# ----------------------------------------------------------------------------
# Adam / AdamW, one tensor                        optimi/adam.py:354-396
# ----------------------------------------------------------------------------
def adam_tensor(param, grad, exp_avg, exp_avg_sq, kahan_comp, *, lr, beta1_comp, beta2_hat, beta2_comp,
                weight_decay, eps, decouple_wd, kahan_sum=False, update_parameters=True):
    """``weight_decay`` is the already-formed factor (1 - lr*wd) when decoupled, the raw
    coefficient for L2  (optimi/adam.py:268-273)."""
    if weight_decay != 0 and update_parameters:  # adam.py:373-377
        if decouple_wd:
            param.mul_(weight_decay)
        else:
            grad.add_(param, alpha=weight_decay)

    exp_avg.lerp_(grad, weight=beta1_comp)  # adam.py:380
    exp_avg_sq.mul_(beta2_hat).addcmul_(grad, grad, value=beta2_comp)  # adam.py:381

    if not update_parameters:  # adam.py:383
        return
    denom = exp_avg_sq.sqrt().add_(eps)
    if kahan_sum and param.dtype in LOW_PRECISION:  # adam.py:384-393
        kahan_comp.addcdiv_(exp_avg, denom, value=-lr)
        _kahan_commit(param, grad, kahan_comp)
    else:  # adam.py:396
        param.addcdiv_(exp_avg, denom, value=-lr)


def adam(params, grads, exp_avgs, exp_avg_sqs, kahan_comps=None, *, lr, beta1, beta2, weight_decay, eps, step,
         decouple_wd, decouple_lr=False, max_lr=None, kahan_sum=False, optimizer_accumulation=False, **_):
    """Functional Adam/AdamW step over a tensor or a list  (optimi/adam.py:213-309)."""
    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    if weight_decay != 0:  # adam.py:269-273
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    params, grads, exp_avgs, exp_avg_sqs = map(_as_list, (params, grads, exp_avgs, exp_avg_sqs))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, v, k in zip(params, grads, exp_avgs, exp_avg_sqs, kahan_comps):
        adam_tensor(p, g, m, v, k, lr=lr, beta1_comp=1 - beta1_hat, beta2_hat=beta2_hat, beta2_comp=1 - beta2_hat,
                    weight_decay=weight_decay, eps=eps, decouple_wd=(decouple_wd or decouple_lr), kahan_sum=kahan_sum,
                    update_parameters=not optimizer_accumulation)


def adamw(params, grads, exp_avgs, exp_avg_sqs, kahan_comps=None, **kw):
    """AdamW = Adam with ``decouple_wd=True``  (optimi/adamw.py:123-143)."""
    kw["decouple_wd"] = True
    adam(params, grads, exp_avgs, exp_avg_sqs, kahan_comps, **kw)


# ----------------------------------------------------------------------------
# Lion, one tensor                                optimi/lion.py:301-338
# ----------------------------------------------------------------------------
def lion_tensor(param, grad, exp_avg, kahan_comp, *, lr, beta1_comp, beta2_comp, weight_decay, kahan_sum=False,
                update_parameters=True):
    if weight_decay != 0 and update_parameters:  # lion.py:314-315
        param.mul_(weight_decay)
    if update_parameters:  # lion.py:318-319
        update = exp_avg.lerp(grad, weight=beta1_comp).sign_()
    exp_avg.lerp_(grad, weight=beta2_comp)  # lion.py:322
    if not update_parameters:
        return
    if kahan_sum and param.dtype in LOW_PRECISION:  # lion.py:325-335
        kahan_comp.add_(update, alpha=-lr)
        _kahan_commit(param, grad, kahan_comp)
    else:  # lion.py:338
        param.add_(update, alpha=-lr)


def lion(params, grads, exp_avgs, kahan_comps=None, *, lr, beta1, beta2, weight_decay, decouple_lr=False, max_lr=None,
         kahan_sum=False, optimizer_accumulation=False, **_):
    """Functional Lion step  (optimi/lion.py:187-266).  No step counter, no debiasing."""
    if weight_decay != 0:  # lion.py:226-231
        weight_decay = 1 - (lr / max_lr) * weight_decay if decouple_lr else 1 - lr * weight_decay
    params, grads, exp_avgs = map(_as_list, (params, grads, exp_avgs))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, k in zip(params, grads, exp_avgs, kahan_comps):
        lion_tensor(p, g, m, k, lr=lr, beta1_comp=1 - beta1, beta2_comp=1 - beta2, weight_decay=weight_decay,
                    kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation)


# ----------------------------------------------------------------------------
# StableAdamW, one tensor                         optimi/stableadamw.py:421-472
# ----------------------------------------------------------------------------
def stableadamw_tensor(param, grad, exp_avg, exp_avg_sq, eps_sq, kahan_comp, *, lr, beta1_comp, beta2_hat, beta2_comp,
                       weight_decay, eps, decouple_lr, max_lr, kahan_sum=False, update_parameters=True):
    """``weight_decay`` is the raw coefficient; the factor is formed from the clipped lr.
    ``eps_sq`` is a 0-dim tensor in the param dtype (optimi/stableadamw.py:119)."""
    exp_avg.lerp_(grad, weight=beta1_comp)  # stableadamw.py:442
    exp_avg_sq.mul_(beta2_hat).addcmul_(grad, grad, value=beta2_comp)  # stableadamw.py:443
    if not update_parameters:
        return
    rms = grad.pow(2).div_(exp_avg_sq.maximum(eps_sq)).mean().sqrt()  # stableadamw.py:447
    lr = lr / max(1, rms.item())  # stableadamw.py:450
    if weight_decay != 0:  # stableadamw.py:453-458
        factor = 1 - (lr / max_lr) * weight_decay if decouple_lr else 1 - lr * weight_decay
        param.mul_(factor)
    denom = exp_avg_sq.sqrt().add_(eps)
    if kahan_sum and param.dtype in LOW_PRECISION:  # stableadamw.py:460-469
        kahan_comp.addcdiv_(exp_avg, denom, value=-lr)
        _kahan_commit(param, grad, kahan_comp)
    else:  # stableadamw.py:472
        param.addcdiv_(exp_avg, denom, value=-lr)


def make_eps_sq(param: Tensor, eps: float) -> Tensor:
    """0-dim eps**2 in the param dtype, as the reference keeps in state (stableadamw.py:119)."""
    return torch.tensor(eps**2, dtype=param.dtype, device=param.device)


def stableadamw(params, grads, exp_avgs, exp_avg_sqs, eps_sqs, kahan_comps=None, *, lr, beta1, beta2, weight_decay,
                eps, step, decouple_lr=False, max_lr=None, kahan_sum=False, optimizer_accumulation=False, **_):
    """Functional StableAdamW step  (optimi/stableadamw.py:277-371)."""
    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    params, grads, exp_avgs, exp_avg_sqs, eps_sqs = map(_as_list, (params, grads, exp_avgs, exp_avg_sqs, eps_sqs))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, v, e2, k in zip(params, grads, exp_avgs, exp_avg_sqs, eps_sqs, kahan_comps):
        stableadamw_tensor(p, g, m, v, e2, k, lr=lr, beta1_comp=1 - beta1_hat, beta2_hat=beta2_hat,
                           beta2_comp=1 - beta2_hat, weight_decay=weight_decay, eps=eps, decouple_lr=decouple_lr,
                           max_lr=max_lr, kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation)


# ----------------------------------------------------------------------------
# Adan, one tensor                                optimi/adan.py:405-469
# ----------------------------------------------------------------------------
def adan_tensor(param, grad, exp_avg, exp_avg_diff, exp_avg_sq, prev_grad, kahan_comp, *, lr, beta1_comp, beta2,
                beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, adam_wd, kahan_sum=False, update_parameters=True):
    """``weight_decay`` is the formed factor: 1 + lr*wd (Adan style) or 1 - lr*wd (``adam_wd``)
    (optimi/adan.py:300-309).  ``prev_grad`` holds the negated previous gradient."""
    prev_grad.add_(grad)  # adan.py:427   g_k - g_{k-1}
    exp_avg.lerp_(grad, weight=beta1_comp)  # adan.py:430
    exp_avg_diff.lerp_(prev_grad, weight=beta2_comp)  # adan.py:433
    prev_grad.mul_(beta2).add_(grad)  # adan.py:436
    exp_avg_sq.mul_(beta3_hat).addcmul_(prev_grad, prev_grad, value=beta3_comp)  # adan.py:437
    prev_grad.copy_(grad).mul_(-1)  # adan.py:440
    if not update_parameters:
        return
    denom = exp_avg_sq.sqrt().add_(eps)  # adan.py:444
    if adam_wd and weight_decay != 0:  # adan.py:447-448
        param.mul_(weight_decay)
    if kahan_sum and param.dtype in LOW_PRECISION:  # adan.py:450-458
        kahan_comp.addcdiv_(exp_avg, denom, value=-lr)
        kahan_comp.addcdiv_(exp_avg_diff, denom, value=-lr * beta2)
        _kahan_commit(param, grad, kahan_comp)
    else:  # adan.py:461-462
        param.addcdiv_(exp_avg, denom, value=-lr)
        param.addcdiv_(exp_avg_diff, denom, value=-lr * beta2)
    if not adam_wd and weight_decay != 0:  # adan.py:465-466
        param.div_(weight_decay)


def adan_first_prev_grad(grad: Tensor) -> Tensor:
    """State created on a tensor's first step: the negated gradient (optimi/adan.py:109)."""
    return grad.clone().mul_(-1)


def adan(params, grads, exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads, kahan_comps=None, *, lr, beta1, beta2, beta3,
         weight_decay, eps, step, decouple_lr=False, max_lr=None, adam_wd=False, kahan_sum=False,
         optimizer_accumulation=False, **_):
    """Functional Adan step  (optimi/adan.py:236-350)."""
    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    beta3_hat = debias_beta(beta3, t)
    if weight_decay != 0:  # adan.py:300-309
        weight_decay = (lr / max_lr) * weight_decay if decouple_lr else lr * weight_decay
        weight_decay = 1 - weight_decay if adam_wd else 1 + weight_decay
    params, grads, exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads = map(
        _as_list, (params, grads, exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, df, n, pg, k in zip(params, grads, exp_avgs, exp_avg_diffs, exp_avg_sqs, prev_grads, kahan_comps):
        adan_tensor(p, g, m, df, n, pg, k, lr=lr, beta1_comp=1 - beta1_hat, beta2=beta2, beta2_comp=1 - beta2_hat,
                    beta3_hat=beta3_hat, beta3_comp=1 - beta3_hat, eps=eps, weight_decay=weight_decay, adam_wd=adam_wd,
                    kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation)


# ----------------------------------------------------------------------------
# SGD, one tensor                                 optimi/sgd.py:329-372
# ----------------------------------------------------------------------------
def sgd_tensor(param, grad, exp_avg, kahan_comp, *, lr, momentum, weight_decay, dampening, decouple_wd,
               kahan_sum=False, update_parameters=True):
    if weight_decay != 0 and update_parameters:  # sgd.py:343-347
        if decouple_wd:
            param.mul_(weight_decay)
        else:
            grad.add_(param, alpha=weight_decay)
    if momentum != 0:  # sgd.py:349-357
        if dampening:
            exp_avg.lerp_(grad, weight=1 - momentum)
        else:
            exp_avg.mul_(momentum).add_(grad)
    else:
        exp_avg = grad
    if not update_parameters:
        return
    if kahan_sum and param.dtype in LOW_PRECISION:  # sgd.py:360-369
        kahan_comp.add_(exp_avg, alpha=-lr)
        _kahan_commit(param, grad, kahan_comp)
    else:  # sgd.py:372
        param.add_(exp_avg, alpha=-lr)


def sgd(params, grads, exp_avgs, kahan_comps=None, *, lr, momentum, weight_decay, dampening, decouple_wd,
        decouple_lr=False, max_lr=None, kahan_sum=False, optimizer_accumulation=False, **_):
    """Functional SGD step  (optimi/sgd.py:213-298)."""
    if weight_decay != 0:  # sgd.py:256-260
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    params, grads, exp_avgs = map(_as_list, (params, grads, exp_avgs))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, k in zip(params, grads, exp_avgs, kahan_comps):
        sgd_tensor(p, g, m, k, lr=lr, momentum=momentum, weight_decay=weight_decay, dampening=dampening,
                   decouple_wd=(decouple_wd or decouple_lr), kahan_sum=kahan_sum,
                   update_parameters=not optimizer_accumulation)


# ----------------------------------------------------------------------------
# RAdam and Ranger, one tensor          optimi/radam.py:368-417, ranger.py:402-473
# ----------------------------------------------------------------------------
def rectification(beta2: float, step: int):
    """Variance rectification term, or None while the approximated SMA is too short
    (optimi/radam.py:269-277, ranger.py:290-298)."""
    rho_inf = 2 / (1 - beta2) - 1
    rho = rho_inf - 2 * step * (beta2**step) / (1 - beta2**step)
    if rho > 5:
        return math.sqrt(((rho - 4) * (rho - 2) * rho_inf) / ((rho_inf - 4) * (rho_inf - 2) * rho))
    return None


def _radam_step(target, exp_avg, exp_avg_sq, *, lr, eps, rect):
    """target += -lr*rect*m/(sqrt(v)+eps) once rectified, else -lr*m  (radam.py:398-417)."""
    if rect is not None:
        target.addcdiv_(exp_avg, exp_avg_sq.sqrt().add_(eps), value=-lr * rect)
    else:
        target.add_(exp_avg, alpha=-lr)


def radam_tensor(param, grad, exp_avg, exp_avg_sq, kahan_comp, *, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay,
                 eps, rect, decouple_wd, kahan_sum=False, update_parameters=True):
    if weight_decay != 0 and update_parameters:  # radam.py:387-391
        if decouple_wd:
            param.mul_(weight_decay)
        else:
            grad.add_(param, alpha=weight_decay)
    exp_avg.lerp_(grad, weight=beta1_comp)  # radam.py:394
    exp_avg_sq.mul_(beta2_hat).addcmul_(grad, grad, value=beta2_comp)  # radam.py:395
    if not update_parameters:
        return
    if kahan_sum and param.dtype in LOW_PRECISION:  # radam.py:398-410
        _radam_step(kahan_comp, exp_avg, exp_avg_sq, lr=lr, eps=eps, rect=rect)
        _kahan_commit(param, grad, kahan_comp)
    else:  # radam.py:412-417
        _radam_step(param, exp_avg, exp_avg_sq, lr=lr, eps=eps, rect=rect)


def ranger_tensor(param, grad, exp_avg, exp_avg_sq, la_param, kahan_comp, *, lr, beta1_comp, beta2_hat, beta2_comp,
                  weight_decay, eps, rect, k, alpha, step, decouple_wd, kahan_sum=False, update_parameters=True):
    """RAdam step, then every ``k``-th step the Lookahead interpolation with the slow weights."""
    radam_tensor(param, grad, exp_avg, exp_avg_sq, kahan_comp, lr=lr, beta1_comp=beta1_comp, beta2_hat=beta2_hat,
                 beta2_comp=beta2_comp, weight_decay=weight_decay, eps=eps, rect=rect, decouple_wd=decouple_wd,
                 kahan_sum=kahan_sum, update_parameters=update_parameters)
    if not update_parameters or step % k != 0:
        return
    if kahan_sum and param.dtype in LOW_PRECISION:  # ranger.py:452-463
        kahan_comp.add_(param.sub_(la_param), alpha=alpha)
        grad.copy_(la_param.detach())
        la_param.add_(kahan_comp)
        kahan_comp.add_(grad.sub_(la_param), alpha=alpha)
        param.copy_(la_param)
    else:  # ranger.py:471-473
        la_param.add_(param.sub(la_param), alpha=alpha)
        param.copy_(la_param)


def _radam_prologue(lr, beta1, beta2, weight_decay, step, decouple_wd, decouple_lr, max_lr):
    t = _tick(step)
    beta1_hat = debias_beta(beta1, t)
    beta2_hat = debias_beta(beta2, t)
    rect = rectification(beta2, t)
    if weight_decay != 0:
        if decouple_lr:
            weight_decay = 1 - (lr / max_lr) * weight_decay
        elif decouple_wd:
            weight_decay = 1 - lr * weight_decay
    return t, beta1_hat, beta2_hat, rect, weight_decay


def radam(params, grads, exp_avgs, exp_avg_sqs, kahan_comps=None, *, lr, beta1, beta2, weight_decay, eps, step,
          decouple_wd, decouple_lr=False, max_lr=None, kahan_sum=False, optimizer_accumulation=False, **_):
    """Functional RAdam step  (optimi/radam.py:214-322)."""
    _, b1h, b2h, rect, weight_decay = _radam_prologue(lr, beta1, beta2, weight_decay, step, decouple_wd, decouple_lr, max_lr)
    params, grads, exp_avgs, exp_avg_sqs = map(_as_list, (params, grads, exp_avgs, exp_avg_sqs))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, v, kc in zip(params, grads, exp_avgs, exp_avg_sqs, kahan_comps):
        radam_tensor(p, g, m, v, kc, lr=lr, beta1_comp=1 - b1h, beta2_hat=b2h, beta2_comp=1 - b2h,
                     weight_decay=weight_decay, eps=eps, rect=rect, decouple_wd=(decouple_wd or decouple_lr),
                     kahan_sum=kahan_sum, update_parameters=not optimizer_accumulation)


def ranger(params, grads, exp_avgs, exp_avg_sqs, la_params, kahan_comps=None, *, lr, beta1, beta2, weight_decay, eps,
           k, alpha, step, decouple_wd, decouple_lr=False, max_lr=None, kahan_sum=False, optimizer_accumulation=False,
           **_):
    """Functional Ranger step  (optimi/ranger.py:230-344)."""
    t, b1h, b2h, rect, weight_decay = _radam_prologue(lr, beta1, beta2, weight_decay, step, decouple_wd, decouple_lr, max_lr)
    params, grads, exp_avgs, exp_avg_sqs, la_params = map(_as_list, (params, grads, exp_avgs, exp_avg_sqs, la_params))
    kahan_comps = [None] * len(params) if kahan_comps is None else _as_list(kahan_comps)
    for p, g, m, v, la, kc in zip(params, grads, exp_avgs, exp_avg_sqs, la_params, kahan_comps):
        ranger_tensor(p, g, m, v, la, kc, lr=lr, beta1_comp=1 - b1h, beta2_hat=b2h, beta2_comp=1 - b2h,
                      weight_decay=weight_decay, eps=eps, rect=rect, k=k, alpha=alpha, step=t,
                      decouple_wd=(decouple_wd or decouple_lr), kahan_sum=kahan_sum,
                      update_parameters=not optimizer_accumulation)


# ----------------------------------------------------------------------------
# A minimal stateful driver: what the reference's optimizer classes do around
# the functional call (lazy state, step counters, Kahan tri-state), reduced to
# plain lists so tests and the CPU baseline can run whole synthetic lists.
# ----------------------------------------------------------------------------
class ForLoopRun:
    """Holds states for a list of tensors and steps them with one of the functional forms.

    ``name`` in {"adam", "adamw", "lion", "stableadamw", "adan"}.  Mirrors
    ``_init_state`` of the reference classes (adam.py:95-109, lion.py:89-99,
    stableadamw.py:115-133, adan.py:104-120): zero states in the param dtype, a Kahan
    buffer only for low-precision params when ``kahan_sum`` is True or None (Adan: only
    when True, adan.py:72), Adan's ``prev_grad`` seeded with the negated first gradient,
    and one step counter per group or – in gradient-release mode – per tensor.
    """

    # constructor defaults of the reference classes (adam.py:56-70, adamw.py:48-61, lion.py:56-68,
    # stableadamw.py:76-89, adan.py:62-76); ``lr`` is always required
    DEFAULTS = {
        "adam": dict(betas=(0.9, 0.99), weight_decay=0.0, eps=1e-6, decouple_wd=False),
        "adamw": dict(betas=(0.9, 0.99), weight_decay=1e-2, eps=1e-6),
        "lion": dict(betas=(0.9, 0.99), weight_decay=0.0),
        "stableadamw": dict(betas=(0.9, 0.99), weight_decay=1e-2, eps=1e-6),
        "adan": dict(betas=(0.98, 0.92, 0.99), weight_decay=2e-2, eps=1e-6),
        "sgd": dict(momentum=0.0, weight_decay=0.0, dampening=False, decouple_wd=False, torch_init=False),
        "radam": dict(betas=(0.9, 0.99), weight_decay=0.0, eps=1e-6, decouple_wd=False),
        "ranger": dict(betas=(0.9, 0.99), weight_decay=0.0, eps=1e-6, k=6, alpha=0.5, decouple_wd=True),
    }

    def __init__(self, name, params, *, gradient_release=False, functional=False, **hyper):
        self.name = name
        self.params = list(params)
        self.gradient_release = gradient_release
        # functional=True drives the functional form the way a direct caller does rather than the
        # way the reference's classes do.  The one difference: Adan's ``adam_wd`` reaches the
        # functional form (the class never forwards it, adan.py:181-203, and clears it when Kahan
        # summation is on, adan.py:156-157).
        self.functional = functional
        self.hyper = {**self.DEFAULTS[name], **hyper}
        if self.hyper.get("decouple_lr") and self.hyper.get("max_lr") is None:
            self.hyper["max_lr"] = self.hyper["lr"]  # optimizer.py:20-21
        ks = self.hyper.pop("kahan_sum", False if name == "adan" else None)
        self.kahan = [(ks or ks is None) and p.dtype in LOW_PRECISION for p in self.params]
        self.kahan_sum = any(self.kahan) or bool(ks)
        if name == "adan" and self.kahan_sum and not functional:
            self.hyper["adam_wd"] = False  # adan.py:156-157
        self.state = [None] * len(self.params)
        self.group_step = torch.tensor(0, dtype=torch.int32)
        self.optimizer_accumulation = False

    def _ensure_state(self, i, grad):
        if self.state[i] is not None:
            return self.state[i]
        p = self.params[i]
        st = {"exp_avg": torch.zeros_like(p)}
        if self.name == "sgd":  # sgd.py:97-107
            h = self.hyper
            if h["dampening"] and h["torch_init"]:
                st["exp_avg"] = grad.detach().clone()
                if h["weight_decay"] != 0 and not h.get("decouple_lr") and not h["decouple_wd"]:
                    st["exp_avg"].add_(p, alpha=h["weight_decay"])
            elif h["momentum"] == 0:
                st["exp_avg"] = None
        if self.name in ("adam", "adamw", "stableadamw", "adan", "radam", "ranger"):
            st["exp_avg_sq"] = torch.zeros_like(p)
        if self.name == "ranger":
            st["la_param"] = p.detach().clone()  # ranger.py:142
        if self.name == "stableadamw":
            st["eps_sq"] = make_eps_sq(p, self.hyper["eps"])
        if self.name == "adan":
            st["exp_avg_diff"] = torch.zeros_like(p)
            st["prev_grad"] = adan_first_prev_grad(grad)
        st["kahan_comp"] = torch.zeros_like(p) if self.kahan[i] else None
        st["step"] = torch.tensor(0, dtype=torch.int32)
        self.state[i] = st
        return st

    def _call(self, idxs, grads, step, accumulate):
        sts = [self._ensure_state(i, g) for i, g in zip(idxs, grads)]
        ps = [self.params[i] for i in idxs]
        col = lambda key: [s[key] for s in sts]  # noqa: E731
        h = dict(self.hyper)
        common = dict(step=step, kahan_sum=self.kahan_sum, optimizer_accumulation=accumulate)
        if self.name in ("adam", "adamw"):
            b1, b2 = h.pop("betas", (0.9, 0.99))
            if self.name == "adam":
                h.setdefault("decouple_wd", False)
            self._invoke(self.name, [ps, grads, col("exp_avg"), col("exp_avg_sq"), col("kahan_comp")],
                         dict(beta1=b1, beta2=b2, **h, **common))
        elif self.name == "lion":
            b1, b2 = h.pop("betas", (0.9, 0.99))
            common.pop("step")
            self._invoke("lion", [ps, grads, col("exp_avg"), col("kahan_comp")], dict(beta1=b1, beta2=b2, **h, **common))
        elif self.name == "stableadamw":
            b1, b2 = h.pop("betas", (0.9, 0.99))
            self._invoke("stableadamw", [ps, grads, col("exp_avg"), col("exp_avg_sq"), col("eps_sq"), col("kahan_comp")],
                         dict(beta1=b1, beta2=b2, **h, **common))
        elif self.name == "adan":
            b1, b2, b3 = h.pop("betas", (0.98, 0.92, 0.99))
            # the reference class never forwards adam_wd (adan.py:181-203): always Adan-style decay
            adam_wd = bool(h.pop("adam_wd", False)) and self.functional
            self._invoke("adan", [ps, grads, col("exp_avg"), col("exp_avg_diff"), col("exp_avg_sq"), col("prev_grad"),
                                  col("kahan_comp")], dict(beta1=b1, beta2=b2, beta3=b3, adam_wd=adam_wd, **h, **common))
        elif self.name == "sgd":
            common.pop("step")
            h.pop("torch_init", None)
            self._invoke("sgd", [ps, grads, col("exp_avg"), col("kahan_comp")], dict(**h, **common))
        elif self.name == "radam":
            b1, b2 = h.pop("betas")
            self._invoke("radam", [ps, grads, col("exp_avg"), col("exp_avg_sq"), col("kahan_comp")],
                         dict(beta1=b1, beta2=b2, **h, **common))
        elif self.name == "ranger":
            b1, b2 = h.pop("betas")
            self._invoke("ranger", [ps, grads, col("exp_avg"), col("exp_avg_sq"), col("la_param"), col("kahan_comp")],
                         dict(beta1=b1, beta2=b2, **h, **common))
        else:
            raise ValueError(self.name)

    def _invoke(self, form, columns, kwargs):
        """Calls the functional form ``form`` of this module on the tensor columns (params, grads, the
        states, the Kahan buffers, in the form's positional order).  A subclass can hand the same
        arguments to another implementation with the same signatures."""
        globals()[form](*columns, **kwargs)

    def step(self, grads):
        """Whole-list step with one shared counter (adam.py:158-182).  ``grads[i] is None`` skips tensor i."""
        idxs = [i for i, g in enumerate(grads) if g is not None]
        self._call(idxs, [grads[i] for i in idxs], self.group_step, False)

    def step_param(self, i, grad):
        """Per-tensor gradient-release step with that tensor's own counter (adam.py:183-208)."""
        st = self._ensure_state(i, grad)
        self._call([i], [grad], st["step"], self.optimizer_accumulation)
