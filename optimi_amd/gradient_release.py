"""Gradient release: each parameter is stepped the moment autograd has finished accumulating
its gradient, and the gradient is freed right after, so a full set of gradients never exists
at once.  Same entry points and error behaviour as optimi/gradientrelease.py:13-61; the hook
itself is native (see ``OptimiOptimizer._native_hook``)."""

from __future__ import annotations

import warnings

import torch

from .optimizers import OptimiOptimizer

__all__ = ["prepare_for_gradient_release", "remove_gradient_release"]

_HOOKS_ATTR = "_gradient_release_hooks"
_OPTIMIZER_ATTR = "_gradient_release_optimizer"


def _gradient_release_hook(param: torch.Tensor, optimizer: OptimiOptimizer):
    """Python form of the hook, kept as the definition of what the native hook must do (the
    tests run the two side by side): step this parameter, then drop its gradient
    (optimi/gradientrelease.py:13-15)."""
    optimizer._release(param)


def _has_foreign_hooks(param: torch.Tensor) -> bool:
    hooks = param._post_accumulate_grad_hooks
    return hooks is not None and len(hooks) > 0


def prepare_for_gradient_release(model: torch.nn.Module, optimizer: OptimiOptimizer, ignore_existing_hooks: bool = False):
    """Attach the gradient-release step to every trainable parameter of ``model``.

    ``optimizer`` must be an optimi_amd optimizer constructed with ``gradient_release=True``
    (``TypeError`` / ``ValueError`` otherwise).  A parameter that already carries a
    post-accumulate-grad hook is an error - nothing is registered then - unless
    ``ignore_existing_hooks`` is set.  Undo with ``remove_gradient_release``.
    """
    if not isinstance(optimizer, OptimiOptimizer):
        raise TypeError("`optimizer` must be an instance of `OptimiOptimizer`")
    if not optimizer.defaults["gradient_release"]:
        raise ValueError("`optimizer` must be initialized with `gradient_release=True`")

    trainable = [p for p in model.parameters() if p.requires_grad]
    if not ignore_existing_hooks and any(_has_foreign_hooks(p) for p in trainable):
        raise ValueError(
            "Model already has post_accumulate_grad_hooks. If this is expected, rerun with `ignore_existing_hooks=True`."
        )

    hook = optimizer._native_hook()  # one callable for all parameters
    setattr(model, _HOOKS_ATTR, [p.register_post_accumulate_grad_hook(hook) for p in trainable])
    # the native hook refers to its optimizer weakly; the model keeps the optimizer alive for as
    # long as the hooks are in place, which is what the reference's closures do implicitly
    setattr(model, _OPTIMIZER_ATTR, optimizer)


def remove_gradient_release(model: torch.nn.Module):
    """Detach the hooks ``prepare_for_gradient_release`` put on ``model``'s parameters; warns if
    there are none."""
    handles = getattr(model, _HOOKS_ATTR, None)
    if handles is None:
        warnings.warn("`model` does not have any gradient release post_accumulate_grad_hooks to remove.")
        return
    for handle in handles:
        handle.remove()
    delattr(model, _HOOKS_ATTR)
    if hasattr(model, _OPTIMIZER_ATTR):
        delattr(model, _OPTIMIZER_ATTR)
