"""Scalar helpers of the step prologue (Python doubles, as in the reference) and the two
model-preparation helpers that decide which tensors land in which launch: the decay /
no-decay split of a model's parameters and the low-precision cast that keeps chosen
modules and buffers in float32."""

from __future__ import annotations

from typing import Any, Iterable

import torch
from torch import nn


def debias(beta: float, step: int) -> float:
    """Adam-style debias term ``1 - beta**step``  (optimi/utils.py:26-28)."""
    return 1 - beta**step


def debias_beta(beta: float, step: int) -> float:
    """Beta with the debias correction folded in, ``(beta**t - beta) / (beta**t - 1)``,
    equal to ``beta * (1 - beta**(t-1)) / (1 - beta**t)``  (optimi/utils.py:31-36)."""
    bt = beta**step
    return (bt - beta) / (bt - 1)


def param_groups_weight_decay(model: nn.Module, weight_decay: float = 1e-2,
                              additional_layers: Iterable[str] | None = None) -> list[dict[str, Any]]:
    """Two parameter groups: biases, 0-d/1-d tensors (normalization weights) and any parameter
    whose name contains one of ``additional_layers`` get ``weight_decay=0``; all other trainable
    parameters get ``weight_decay``.  Each group is stepped as one launch, whatever dtypes it holds.
    (optimi/utils.py:41-71; order of the groups as there: no-decay first.)"""
    skip = tuple(additional_layers) if additional_layers is not None else ()
    groups = {False: [], True: []}
    for name, param in model.named_parameters():
        if param.requires_grad:
            exempt = param.ndim <= 1 or name.endswith(".bias") or any(s in name for s in skip)
            groups[not exempt].append(param)
    return [{"params": groups[False], "weight_decay": 0.0}, {"params": groups[True], "weight_decay": weight_decay}]


def _as_tuple(x) -> tuple:
    if x is None:
        return ()
    if isinstance(x, (str, type)):
        return (x,)
    if not isinstance(x, Iterable):
        return (x,)
    return tuple(x)


def _is_module_type(x) -> bool:
    return isinstance(x, type) and issubclass(x, nn.Module)


def to_low_precision(model: nn.Module, dtype: torch.dtype = torch.bfloat16, device: torch.device | str | None = None,
                     fp32_modules=nn.Embedding, fp32_buffers=("rope", "rotary")) -> nn.Module:
    """Casts ``model`` in place to ``dtype`` (and moves it to ``device`` if given), except:

    * modules that are instances of ``fp32_modules`` (default ``nn.Embedding``) keep their own
      parameters and buffers in float32;
    * modules whose qualified name contains one of the strings in ``fp32_buffers`` (default
      "rope", "rotary"), or that are instances of a module type listed there, keep their own
      buffers in float32 (their parameters are cast).

    Non-floating-point tensors are left alone.  The optimizers step each of the resulting mixed
    bf16 / fp32 parameter groups as one launch.  (optimi/utils.py:104-169)"""
    mod_types = _as_tuple(fp32_modules)
    if not all(_is_module_type(t) for t in mod_types):
        raise TypeError("fp32_modules must be nn.Module subclass type(s)")
    keywords, buf_types = [], []
    for item in _as_tuple(fp32_buffers):
        if isinstance(item, str):
            keywords.append(item.lower())
        elif _is_module_type(item):
            buf_types.append(item)
        else:
            raise TypeError("fp32_buffers items must be str or a nn.Module subclass type")
    buf_types = tuple(buf_types)

    for qual, module in model.named_modules(remove_duplicate=True):
        params_fp32 = isinstance(module, mod_types) if mod_types else False
        buffers_fp32 = params_fp32 or any(k in qual for k in keywords) or (bool(buf_types) and isinstance(module, buf_types))
        own_params = {id(p) for p in module._parameters.values() if p is not None}
        own_params |= {id(p.grad) for p in module._parameters.values() if p is not None and p.grad is not None}
        own_buffers = {id(b) for b in module._buffers.values() if b is not None}

        def cast(t: torch.Tensor, own_params=own_params, own_buffers=own_buffers, params_fp32=params_fp32,
                 buffers_fp32=buffers_fp32):
            if not t.is_floating_point():
                return t
            if id(t) in own_params:
                return t.to(dtype=torch.float32 if params_fp32 else dtype, device=device)
            if id(t) in own_buffers:
                return t.to(dtype=torch.float32 if buffers_fp32 else dtype, device=device)
            return t

        # Module._apply swaps parameters the way .to() does and passes their gradients through
        # the same function, so a gradient follows its parameter's dtype
        module._apply(cast, recurse=False)
    return model
