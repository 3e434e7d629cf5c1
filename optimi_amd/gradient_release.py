"""Gradient release: run the optimizer step for a parameter as soon as its gradient has been
accumulated, then free the gradient (optimi/gradientrelease.py:13-61)."""

from __future__ import annotations

from warnings import warn

from torch import Tensor
from torch.nn import Module

from .optimizers import OptimiOptimizer

__all__ = ["prepare_for_gradient_release", "remove_gradient_release"]


def _gradient_release_hook(param: Tensor, optimizer: OptimiOptimizer):
    """What every registered hook does: ``step(param=param)`` then ``zero_grad(param=param)``
    (optimi/gradientrelease.py:13-15).  The hooks registered below are the native form of this
    function (state and group lookup, scalar prologue, launch or parking, freeing the gradient,
    without a Python frame per parameter); this Python form gives the same results."""
    optimizer._release(param)


def prepare_for_gradient_release(model: Module, optimizer: OptimiOptimizer, ignore_existing_hooks: bool = False):
    """Register post_accumulate_grad_hooks on parameters for the gradient release optimization step.

    Args:
        model: Model to register post_accumulate_grad_hooks. Only registers on parameters with
            `requires_grad=True`.
        optimizer: Optimizer providing the fused optimizer step during the backward pass. Requires
            optimizer to be initialized with `gradient_release=True`
        ignore_existing_hooks: If True, ignores existing post_accumulate_grad_hooks on parameters
            and registers gradient release hooks (default: False)
    """
    if not isinstance(optimizer, OptimiOptimizer):
        raise TypeError("`optimizer` must be an instance of `OptimiOptimizer`")
    if not optimizer.defaults["gradient_release"]:
        raise ValueError("`optimizer` must be initialized with `gradient_release=True`")

    hook = optimizer._native_hook()
    registered = []
    for p in model.parameters():
        if not p.requires_grad:
            continue
        existing = p._post_accumulate_grad_hooks
        if existing is not None and len(existing) > 0 and not ignore_existing_hooks:
            for handle in registered:
                handle.remove()
            raise ValueError(
                "Model already has post_accumulate_grad_hooks. If this is expected, rerun with `ignore_existing_hooks=True`."
            )
        registered.append(p.register_post_accumulate_grad_hook(hook))
    model._gradient_release_hooks = registered
    # the hooks refer to the optimizer weakly; the model keeps it alive, as the reference's hooks do
    model._gradient_release_optimizer = optimizer


def remove_gradient_release(model: Module):
    """Removes post_accumulate_grad_hooks created by `prepare_for_gradient_release`.

    Args:
        model: Model to remove gradient release post_accumulate_grad_hooks from.
    """
    if not hasattr(model, "_gradient_release_hooks"):
        warn("`model` does not have any gradient release post_accumulate_grad_hooks to remove.")
        return
    for handle in model._gradient_release_hooks:
        handle.remove()
    del model._gradient_release_hooks
    if hasattr(model, "_gradient_release_optimizer"):
        del model._gradient_release_optimizer
