"""Optimizer classes with the reference's constructor signatures and ``state_dict`` layout.

``OptimiOptimizer`` carries what the reference's base class does (optimi/optimizer.py:12-114):
argument validation, the fully-decoupled weight-decay warning, gradient-release setup, the
``optimizer_accumulation`` switch, and ``step`` / ``zero_grad`` on one parameter.  The step
itself is shared: a subclass only declares its hyper-parameters, its state buffers and which
functional form to call.  Launch workspaces live in ``self._hip_groups``, outside ``state``
and ``param_groups``, so checkpoints hold exactly the reference's keys.
"""

from __future__ import annotations

from collections.abc import Callable, Iterable
from typing import Any
from warnings import warn

import torch
from torch import Tensor
from torch.autograd import Variable
from torch.optim.optimizer import Optimizer

from torch.optim import optimizer as _torch_optimizer

from . import backend
from . import functional as F

__all__ = ["OptimiOptimizer", "Adam", "AdamW", "Lion", "StableAdamW", "Adan", "SGD", "RAdam", "Ranger"]

_LOW_PRECISION = (torch.float16, torch.bfloat16)


def _default_to_fused(params: list[Tensor]) -> bool:
    """The reference picks its accelerated backend when every parameter is a plain floating
    tensor on a bf16-capable GPU (optimi/utils.py:193-201); same rule, HIP devices only."""
    return all(p is None or (type(p) in (Tensor, torch.nn.Parameter) and p.is_cuda and torch.is_floating_point(p))
               for p in params)


def _check_betas(betas):
    for i, b in enumerate(betas):
        if not 0.0 <= b < 1.0:
            raise ValueError(f"Invalid beta{i + 1} parameter: betas[{i}]={b}")


class OptimiOptimizer(Optimizer):
    """Provides common functionality for optimi optimizers."""

    # subclasses fill these in
    _moment_keys: tuple[str, ...] = ()      # zero-initialised buffers shaped like the parameter
    _has_step = True                        # Lion keeps no step counter
    _kahan_placeholder_dtype: torch.dtype | None = torch.uint8  # None: use the parameter dtype (Lion)
    _setup_before_state = False             # StableAdamW resolves its backend before touching state
    _step_state_from_group = True           # per-parameter counter keyed on the group's gradient_release flag (Adan: on the call)
    _release_kind = ""                      # name of the native hook's optimizer kind (KIND_* of the extension)

    # Gradient release parks the steps of tensors with at most this many elements and launches
    # them together - when the parked gradients reach _QUEUE_MAX_BYTES or _QUEUE_MAX_TENSORS, and
    # when the backward pass ends (0 = launch every tensor on its own, from its hook).  Results
    # are identical.  A model with thousands of small tensors steps several times faster, and
    # large matrices do better too: every launch pays a few microseconds to fill and drain the
    # GPU, 7 % of a 45 M-element tensor's step but 1-2 % of a transformer layer's.  The price is
    # that up to _QUEUE_MAX_BYTES of gradients (plus one tensor) stay alive until their launch.
    # Set on the instance, or on the class, before prepare_for_gradient_release.
    native_step = True                      # False: walk the parameters in Python on every step (same results)
    # How a whole-group step reads its tensors.  False: with streaming loads - right for training, where a
    # forward and a backward pass run between two steps and nothing of the optimizer's tensors is left in
    # the GPU's last-level cache.  True: the caller steps back to back with nothing in between (a benchmark
    # loop); if the optimizer's parameters, gradients and states together fit that cache, a step finds them
    # there and reads them with cached loads, 1 % faster then and 8 % slower if the cache was swept after
    # all.  Results are the same either way.
    resident_lists: bool = False
    gradient_release_coalesce = 1 << 26
    _QUEUE_MAX_TENSORS = 1024               # parked steps per launch
    _QUEUE_MAX_BYTES = 128 << 20            # bytes of parked gradients kept alive at most

    def __init__(self, params: Iterable[Tensor] | Iterable[dict], defaults: dict[str, Any]):
        if not 0.0 <= defaults["lr"]:
            raise ValueError(f"Invalid learning rate: lr={defaults['lr']}")
        if not 0.0 <= defaults["weight_decay"]:
            raise ValueError(f"Invalid weight decay: weight_decay={defaults['weight_decay']}")
        if defaults["decouple_lr"] and defaults["max_lr"] is None:
            defaults["max_lr"] = defaults["lr"]
        if defaults["max_lr"] is not None and not 0.0 <= defaults["max_lr"]:
            raise ValueError(f"Invalid maximum learning rate: max_lr={defaults['max_lr']}")
        if defaults["foreach"]:
            # the reference deprecates foreach in favour of its fused backend (optimi/optimizer.py:33-38);
            # here the flag selects the same HIP kernels as triton=True
            warn(
                "Parameter `foreach` is deprecated; optimi_amd serves foreach=True with the fused HIP kernels, as it does "
                "triton=True. Set `foreach=False` or leave it unset to silence this warning.",
                category=DeprecationWarning,
            )
        if defaults["triton"] is False:
            raise ValueError("optimi_amd implements only the fused HIP backend; leave triton unset or pass triton=True")

        super().__init__(params, defaults)

        if self.defaults.get("decouple_lr", False):
            high = [g["weight_decay"] for g in self.param_groups
                    if g.get("decouple_lr", False) and g.get("weight_decay", 0.0) >= 1e-3]
            if high:
                warn(
                    f"You are using weight_decay up to {max(high)} which is potentially high for decouple_lr=True"
                    f". Unlike decoupled weight decay, fully decoupled weight decay does not reduce weight decay by the learning rate.",
                    category=UserWarning,
                )

        self._optimizer_accumulation = False
        self._hip_groups: dict = {}
        self._release_queue = None
        self._release_hook = None
        self._fits_cache = None

        if self.defaults["gradient_release"]:
            if self.defaults["foreach"]:  # optimi/optimizer.py:65-68
                warn("Gradient release (gradient_release=True) and foreach (foreach=True) cannot be used together. "
                     "Disabling foreach.", category=UserWarning)
            self.defaults["foreach"] = False
            for group in self.param_groups:
                group["foreach"] = False
                for p in group["params"]:
                    self.state[p]["group"] = group

    # -- pickling: launch workspaces are device handles, never part of a checkpoint --------
    def __getstate__(self):
        state = super().__getstate__()
        state = dict(state)
        state.pop("_hip_groups", None)
        state.pop("_release_queue", None)
        state.pop("_release_hook", None)
        state.pop("_fits_cache", None)
        return state

    def __setstate__(self, state):
        super().__setstate__(state)
        self.__dict__.setdefault("_hip_groups", {})
        self.__dict__.setdefault("_release_queue", None)
        self.__dict__.setdefault("_release_hook", None)
        self.__dict__["_fits_cache"] = None
        self._invalidate_release_cache()
        self.__dict__.setdefault("_optimizer_accumulation", False)

    def state_dict(self):
        self._flush_release()  # a checkpoint must not miss steps that are still parked
        return super().state_dict()

    @property
    def optimizer_accumulation(self) -> bool:
        "Accumulate gradients in optimizer states during gradient release instead of a full step."
        return self._optimizer_accumulation

    @optimizer_accumulation.setter
    def optimizer_accumulation(self, optimizer_accumulation: bool):
        self._optimizer_accumulation = optimizer_accumulation

    # -- state ---------------------------------------------------------------------------
    def _extra_state(self, group, state, param):
        """Hook for subclasses: state entries beyond the moment buffers."""

    def _init_state(self, group: dict[str, Any], state: dict, param: Tensor, gradient_release: bool | None = None):
        if "kahan_comp" in state:
            return
        for key in self._moment_keys:
            state[key] = torch.zeros_like(param, memory_format=torch.preserve_format)
        self._extra_state(group, state, param)
        if (group["kahan_sum"] or group["kahan_sum"] is None) and param.dtype in _LOW_PRECISION:
            state["kahan_comp"] = torch.zeros_like(param, memory_format=torch.preserve_format)
            group["kahan_sum"] = True
        elif group["triton"]:
            state["kahan_comp"] = torch.zeros(1, dtype=self._kahan_placeholder_dtype or param.dtype, device=param.device)
        else:
            state["kahan_comp"] = None
        self._after_kahan_state(group, state, param)
        release = group["gradient_release"] if self._step_state_from_group else bool(gradient_release)
        if release and self._has_step:
            state["step"] = torch.tensor(0, dtype=torch.int32)

    def _after_kahan_state(self, group, state, param):
        """Hook for subclasses: state entries the reference creates after ``kahan_comp``."""

    def _setup_group(self, group, params):
        if group["setup"]:
            return
        group["setup"] = True
        if self._has_step:
            group["step"] = torch.tensor(0, dtype=torch.int32)
        if group["triton"] is None:
            group["triton"] = _default_to_fused(params)
        self._after_setup(group)

    def _after_setup(self, group):
        """Hook for subclasses."""

    def _collect(self, group):
        """Parameters of ``group`` that have a gradient, with their states created."""
        params = []
        if self._setup_before_state:
            self._setup_group(group, params)
        for p in group["params"]:
            if p.grad is None:
                continue
            params.append(p)
            self._init_state(group, self.state[p], p)
        if not self._setup_before_state:
            self._setup_group(group, params)
        return params

    # -- the step ------------------------------------------------------------------------
    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        raise NotImplementedError

    def step(self, closure: Callable | None = None, param: Tensor | None = None):
        """Performs a single optimization step on the whole model or individual parameter.

        Args:
            closure: A closure which reevaluates the model and returns the loss. Incompatible with
                performing an optimization step on a single `param`.
            param: An individual parameter to perform a fused optimization step during the backward
                pass. Requires optimizer to be initialized with `gradient_release=True` and model
                hooks created with `prepare_for_gradient_release`. Incompatible with `closure`.
        """
        # torch wraps an optimizer's step in a profiler range that runs the step hooks; on a small
        # model that wrapper costs more than the launch.  It is entered here only when it has
        # something to do (a hook is registered, or a profiler is recording).
        if self._has_step_hooks() or torch._C._autograd._profiler_enabled():
            return self._step_with_hooks(closure=closure, param=param)
        loss = self._step(closure=closure, param=param)
        self._optimizer_step_code()
        return loss

    step.hooked = True  # tells torch.optim.Optimizer not to wrap step() itself

    @torch.no_grad()
    def _step(self, closure: Callable | None = None, param: Tensor | None = None):
        loss = None
        if closure is not None and param is None:
            with torch.enable_grad():
                loss = closure()

        if param is None:
            self._flush_release()
            driver = self._driver() if self.native_step else None
            resident = self._lists_are_resident()
            for group in self.param_groups:
                # after a group's first step the whole walk over its parameters is native
                if driver is not None and group["setup"] and driver.step_group(group, resident):
                    continue
                params = self._collect(group)
                if params and not group["triton"]:
                    raise RuntimeError(
                        "optimi_amd: this parameter group cannot use the HIP backend (parameters must be plain "
                        "floating-point tensors on a HIP device) and there is no other backend"
                    )
                states = [self.state[p] for p in params]
                self._functional(group, params, [p.grad for p in params], states, group.get("step"), False, False)
        else:
            state = self.state[param]
            group = state["group"]
            if group["triton"] is None:
                group["triton"] = _default_to_fused([param])
            self._init_state(group, state, param, True)
            if not group["triton"]:
                raise RuntimeError("optimi_amd: parameter is not eligible for the HIP backend and there is no other backend")
            self._functional(group, param, param.grad, state, state.get("step"), True, self._optimizer_accumulation)
        return loss

    _step_with_hooks = Optimizer.profile_hook_step(_step)

    # -- gradient-release fast path --------------------------------------------------------
    def _release_call(self, ext, group, state, param, grad, update, queue):
        """One native call that advances the parameter's step counter, forms the step scalars and
        launches the per-tensor kernel, or parks the step in ``queue`` when the tensor is small
        (then it returns True).  Subclasses forward their hyper-parameters."""
        raise NotImplementedError

    def _has_step_hooks(self) -> bool:
        return bool(self._optimizer_step_pre_hooks or self._optimizer_step_post_hooks
                    or _torch_optimizer._global_optimizer_pre_hooks or _torch_optimizer._global_optimizer_post_hooks)

    @torch.no_grad()
    def _release(self, param: Tensor):
        """``step(param=param)`` followed by ``zero_grad(param=param)``, as the post-accumulate-grad
        hook needs it (optimi/gradientrelease.py:13-15), with the scalar prologue done natively.
        Same results as the public path; it only skips the per-call Python work, which dominates
        when a model has thousands of small tensors.  Falls back to the public methods when step
        hooks are registered, so they still fire."""
        if self._has_step_hooks():
            self.step(param=param)
            self.zero_grad(param=param)
            return
        state = self.state[param]
        group = state["group"]
        if "kahan_comp" not in state:
            if group["triton"] is None:
                group["triton"] = _default_to_fused([param])
            self._init_state(group, state, param, True)
        if not group["triton"]:
            raise RuntimeError("optimi_amd: parameter is not eligible for the HIP backend and there is no other backend")
        backend.check_supported(param)
        parked_or_not = self._release_call(backend.ext(), group, state, param, param.grad, not self._optimizer_accumulation,
                                           self._queue())
        del parked_or_not  # the queue itself arranges for its flush at the end of the backward pass
        param.grad = None

    def _queue(self):
        """The queue that parks the steps of small tensors during a backward pass, or None."""
        if self._release_queue is None and self.gradient_release_coalesce > 0:
            self._release_queue = backend.ext().ReleaseQueue(self.gradient_release_coalesce, self._QUEUE_MAX_TENSORS,
                                                             self._QUEUE_MAX_BYTES)
        return self._release_queue

    def _release_entry(self, param: Tensor):
        """Slow path of the native hook, taken the first time it sees a parameter (and again when
        the parameter's state was replaced): creates the state as ``step(param=param)`` would and
        returns ``(state, group, launch workspace or None)``."""
        state = self.state[param]
        group = state["group"]
        if group["triton"] is None:
            group["triton"] = _default_to_fused([param])
        self._init_state(group, state, param, True)
        if not group["triton"]:
            raise RuntimeError("optimi_amd: parameter is not eligible for the HIP backend and there is no other backend")
        backend.check_supported(param)
        return state, group, self._release_workspace(param)

    def _group_entry(self, param: Tensor, group: dict):
        """Slow path of the native whole-group step, taken the first time it sees a parameter with
        a gradient (and again when its state was replaced): creates the state as ``_collect``
        would and returns ``(state, group, None)``."""
        state = self.state[param]
        self._init_state(group, state, param)
        backend.check_supported(param)
        return state, group, None

    def _release_workspace(self, param: Tensor):
        """Hook for subclasses whose per-tensor step needs device scratch."""
        return None

    def _driver(self):
        """The native driver of this optimizer: the gradient-release hook body and the
        whole-group step, with their per-parameter cache."""
        if self._release_hook is None:
            ext = backend.ext()
            self._release_hook = ext.ReleaseHookCore(self, getattr(ext, self._release_kind), self._queue())
        return self._release_hook

    def _native_hook(self):
        """The post-accumulate-grad hook for this optimizer's parameters: a native callable (one
        per optimizer, shared by its parameters) that does what ``_release`` does."""
        return backend.ext().ReleaseHook(self._driver())

    def _invalidate_release_cache(self):
        self.__dict__["_fits_cache"] = None
        self.__dict__.get("_hip_groups", {}).clear()  # keyed by group dicts that may be gone now
        if self.__dict__.get("_release_hook") is not None:
            self._release_hook.invalidate()

    def _lists_are_resident(self) -> bool:
        """Whether a whole-group step may take its tensors for still being in the last-level cache from
        the step before: the caller has said that it steps back to back (``resident_lists``), and
        everything the optimizer touches in a step - all groups together - fits that cache."""
        if not self.resident_lists:
            return False
        if self._fits_cache is None:
            total = 0
            for group in self.param_groups:
                for p in group["params"]:
                    arrays = 2 + len(self._moment_keys) + (1 if p.dtype in _LOW_PRECISION else 0)
                    total += p.numel() * p.element_size() * arrays
            self._fits_cache = total <= backend.ext().resident_bytes()
        return self._fits_cache

    def _workspaces(self, group: dict) -> dict:
        """The launch workspaces of one parameter group: its device tables then keep this group's list
        from one step to the next, however many other groups the optimizer steps in between."""
        return self._hip_groups.setdefault(id(group), {})

    def load_state_dict(self, state_dict):
        super().load_state_dict(state_dict)
        self._invalidate_release_cache()

    def add_param_group(self, param_group):
        super().add_param_group(param_group)
        self._invalidate_release_cache()

    def _flush_release(self):
        """Launches the gradient-release steps that are still parked."""
        if self._release_queue is not None:
            self._release_queue.flush()

    @torch._disable_dynamo
    def zero_grad(self, set_to_none: bool = True, param: Tensor | None = None):
        """Resets the gradients of all optimized parameters or individual parameter.

        Args:
            set_to_none: If True, the gradients will be deallocated after the call (default: True)
            param: Resets the gradients of the passed `param`. For use with `gradient_release=True`.
        """
        if param is None:
            self._flush_release()
            super().zero_grad(set_to_none=set_to_none)
        elif param.grad is not None:
            if set_to_none:
                param.grad = None
            elif param.grad.grad_fn is not None:
                param.grad.detach_()
            else:
                param.grad.requires_grad_(False)


def _col(states, key):
    """A state entry for one parameter (dict) or the list of it over many (list of dicts)."""
    return states[key] if isinstance(states, dict) else [s[key] for s in states]


class Adam(OptimiOptimizer):
    """Adam optimizer. Optionally with decoupled weight decay (AdamW).

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        betas: Coefficients for gradient and squared gradient moving averages (default: (0.9, 0.99))
        weight_decay: Weight decay coefficient. If `decouple_wd` and `decouple_lr` are False,
            applies L2 penalty (default: 0)
        eps: Added to denominator to improve numerical stability (default: 1e-6)
        decouple_wd: Apply decoupled weight decay instead of L2 penalty (default: False)
        decouple_lr: Apply fully decoupled weight decay instead of L2 penalty (default: False)
        max_lr: Maximum scheduled learning rate. Set if `lr` is not the maximum scheduled learning
            rate and `decouple_lr` is True (default: None)
        kahan_sum: Enables Kahan summation for more accurate parameter updates when training in low
            precision (bfloat16). If unspecified, automatically applies for low precision
            parameters (default: None)
        foreach: Deprecated. True selects the fused HIP kernels, like `triton=True` (default: None)
        triton: Selects the fused backend, here the HIP kernels. Unset or True (default: None)
        gradient_release: Fuses optimizer step and zero_grad as part of the parameter's backward
            pass. Requires model hooks created with `prepare_for_gradient_release`. Incompatible
            with closure (default: False)
    """

    _moment_keys = ("exp_avg", "exp_avg_sq")

    _release_kind = "KIND_ADAM"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 0,
        eps: float = 1e-6,
        decouple_wd: bool = False,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        _check_betas(betas)
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon: {eps=}")
        defaults = dict(lr=lr, beta1=betas[0], beta2=betas[1], eps=eps, weight_decay=weight_decay,
                        decouple_wd=decouple_wd, decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum,
                        foreach=foreach, triton=triton, gradient_release=gradient_release, setup=False)
        super().__init__(params, defaults)

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        F.adam(params, grads, _col(states, "exp_avg"), _col(states, "exp_avg_sq"), _col(states, "kahan_comp"),
               lr=group["lr"], beta1=group["beta1"], beta2=group["beta2"], weight_decay=group["weight_decay"],
               eps=group["eps"], step=step, decouple_wd=group["decouple_wd"], decouple_lr=group["decouple_lr"],
               max_lr=group["max_lr"], kahan_sum=group["kahan_sum"], foreach=False, triton=True,
               gradient_release=gradient_release, optimizer_accumulation=accumulate, _groups=self._workspaces(group), _resident=self._lists_are_resident())


    def _release_call(self, ext, group, state, param, grad, update, queue):
        return ext.adam_release(param, grad, state["exp_avg"], state["exp_avg_sq"], state["kahan_comp"], state["step"], group["lr"],
                         group["beta1"], group["beta2"], group["weight_decay"], group["eps"], group["decouple_wd"],
                         group["decouple_lr"], group["max_lr"], bool(group["kahan_sum"]), update, queue)


class AdamW(Adam):
    """AdamW optimizer: Adam with decoupled weight decay.

    Args as `Adam`, without `decouple_wd` (always on) and with `weight_decay` defaulting to 1e-2.
    """

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 1e-2,
        eps: float = 1e-6,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        super().__init__(params=params, lr=lr, betas=betas, weight_decay=weight_decay, eps=eps, decouple_wd=True,
                         decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum, foreach=foreach, triton=triton,
                         gradient_release=gradient_release)


class Lion(OptimiOptimizer):
    """Lion optimizer. Evolved Sign Momentum.

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        betas: Coefficients for update moving average and gradient moving average (default: (0.9, 0.99))
        weight_decay: Weight decay coefficient. If `decouple_lr` is False, applies decoupled
            weight decay (default: 0)
        decouple_lr: Apply fully decoupled weight decay instead of decoupled weight decay (default: False)
        max_lr: Maximum scheduled learning rate. Set if `lr` is not the maximum scheduled learning
            rate and `decouple_lr` is True (default: None)
        kahan_sum, foreach, triton, gradient_release: as `Adam`
    """

    _moment_keys = ("exp_avg",)
    _has_step = False
    _kahan_placeholder_dtype = None

    _release_kind = "KIND_LION"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 0,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        _check_betas(betas)
        defaults = dict(lr=lr, beta1=betas[0], beta2=betas[1], weight_decay=weight_decay, decouple_lr=decouple_lr,
                        max_lr=max_lr, kahan_sum=kahan_sum, foreach=foreach, triton=triton,
                        gradient_release=gradient_release, setup=False)
        super().__init__(params, defaults)

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        F.lion(params, grads, _col(states, "exp_avg"), _col(states, "kahan_comp"), lr=group["lr"], beta1=group["beta1"],
               beta2=group["beta2"], weight_decay=group["weight_decay"], decouple_lr=group["decouple_lr"],
               max_lr=group["max_lr"], kahan_sum=group["kahan_sum"], foreach=False, triton=True,
               gradient_release=gradient_release, optimizer_accumulation=accumulate, _groups=self._workspaces(group), _resident=self._lists_are_resident())


    def _release_call(self, ext, group, state, param, grad, update, queue):
        return ext.lion_release(param, grad, state["exp_avg"], state["kahan_comp"], group["lr"], group["beta1"], group["beta2"],
                         group["weight_decay"], group["decouple_lr"], group["max_lr"], bool(group["kahan_sum"]), update, queue)


def _restore_scratch_state(optim: OptimiOptimizer):
    """``load_state_dict`` casts floating state to the parameter dtype; bring the fp32 scratch
    back (optimi/stableadamw.py:38-47)."""
    for group in optim.param_groups:
        if group["triton"]:
            for p in group["params"]:
                state = optim.state[p]
                if "mean_square" in state:
                    state["mean_square"] = state["mean_square"].to(dtype=torch.float32, device=p.device)
                else:
                    state["mean_square"] = torch.zeros(1, dtype=torch.float32, device=p.device)


class StableAdamW(OptimiOptimizer):
    """StableAdamW optimizer. An AdamW-Adafactor hybrid with learning rate update clipping.

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        betas: Coefficients for gradient and squared gradient moving averages (default: (0.9, 0.99))
        weight_decay: Weight decay coefficient. If `decouple_lr` is False, applies decoupled weight
            decay (default: 1e-2)
        eps: Added to denominator to improve numerical stability (default: 1e-6)
        decouple_lr, max_lr, kahan_sum, foreach, triton, gradient_release: as `Adam`
    """

    _moment_keys = ("exp_avg", "exp_avg_sq")
    _setup_before_state = True

    _release_kind = "KIND_STABLEADAMW"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 1e-2,
        eps: float = 1e-6,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        _check_betas(betas)
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon: {eps=}")
        defaults = dict(lr=lr, beta1=betas[0], beta2=betas[1], eps=eps, weight_decay=weight_decay,
                        decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum, foreach=foreach, triton=triton,
                        gradient_release=gradient_release, setup=False)
        super().__init__(params, defaults)
        self.register_load_state_dict_post_hook(_restore_scratch_state)

    def _extra_state(self, group, state, param):
        state["eps_sq"] = torch.tensor(group["eps"] ** 2, dtype=param.dtype, device=param.device)

    def _after_kahan_state(self, group, state, param):
        if group["triton"]:
            state["mean_square"] = torch.zeros(1, dtype=torch.float32, device=param.device)

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        F.stableadamw(params, grads, _col(states, "exp_avg"), _col(states, "exp_avg_sq"), _col(states, "eps_sq"),
                      _col(states, "kahan_comp"), lr=group["lr"], beta1=group["beta1"], beta2=group["beta2"],
                      weight_decay=group["weight_decay"], eps=group["eps"], step=step, decouple_lr=group["decouple_lr"],
                      max_lr=group["max_lr"], kahan_sum=group["kahan_sum"], foreach=False, triton=True,
                      gradient_release=gradient_release, optimizer_accumulation=accumulate, mean_squares=None,
                      _groups=self._workspaces(group), _resident=self._lists_are_resident())


    def _release_workspace(self, param):
        return F._workspace(self._hip_groups.setdefault("per_tensor", {}), param.device, param.dtype, "stableadamw_single")

    def _release_call(self, ext, group, state, param, grad, update, queue):
        grp = self._release_workspace(param)
        return ext.stableadamw_release(grp, param, grad, state["exp_avg"], state["exp_avg_sq"], state["kahan_comp"], state["step"],
                                group["lr"], group["beta1"], group["beta2"], group["weight_decay"], group["eps"],
                                group["decouple_lr"], group["max_lr"], bool(group["kahan_sum"]), update, queue)


class Adan(OptimiOptimizer):
    """Adan Optimizer: Adaptive Nesterov Momentum Algorithm.

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        betas: Coefficients for gradient, gradient difference, and squared gradient moving
            averages (default: (0.98, 0.92, 0.99))
        weight_decay: Weight decay coefficient. If `decouple_lr` is False, applies decoupled
            weight decay (default: 2e-2)
        eps: Added to denominator to improve numerical stability (default: 1e-6)
        decouple_lr, max_lr: as `Adam`
        adam_wd: Apply weight decay before parameter update (Adam-style), instead of after the
            update per Adan algorithm (default: False)
        kahan_sum: Enables Kahan summation for low precision parameters (default: False)
        foreach, triton, gradient_release: as `Adam`
    """

    _moment_keys = ("exp_avg", "exp_avg_diff", "exp_avg_sq")
    _step_state_from_group = False

    _release_kind = "KIND_ADAN"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float, float] = (0.98, 0.92, 0.99),
        weight_decay: float = 2e-2,
        eps: float = 1e-6,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        adam_wd: bool = False,
        kahan_sum: bool | None = False,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        _check_betas(betas)
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon: {eps=}")
        defaults = dict(lr=lr, beta1=betas[0], beta2=betas[1], beta3=betas[2], eps=eps, weight_decay=weight_decay,
                        decouple_lr=decouple_lr, max_lr=max_lr, adam_wd=adam_wd, kahan_sum=kahan_sum, foreach=foreach,
                        triton=triton, gradient_release=gradient_release, setup=False)
        super().__init__(params, defaults)

    def _extra_state(self, group, state, param):
        # negated first gradient, so the first difference g_1 - g_0 is zero (optimi/adan.py:109)
        state["prev_grad"] = param.grad.clone().mul_(-1)

    def _after_setup(self, group):
        if group["kahan_sum"]:
            group["adam_wd"] = False

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        # like the reference class, adam_wd is not forwarded: decay is always Adan-style
        # (optimi/adan.py:181-203)
        F.adan(params, grads, _col(states, "exp_avg"), _col(states, "exp_avg_diff"), _col(states, "exp_avg_sq"),
               _col(states, "prev_grad"), _col(states, "kahan_comp"), lr=group["lr"], beta1=group["beta1"],
               beta2=group["beta2"], beta3=group["beta3"], eps=group["eps"], weight_decay=group["weight_decay"],
               step=step, decouple_lr=group["decouple_lr"], max_lr=group["max_lr"], kahan_sum=group["kahan_sum"],
               foreach=False, triton=True, gradient_release=gradient_release,
               optimizer_accumulation=accumulate, _groups=self._workspaces(group), _resident=self._lists_are_resident())

    def _release_call(self, ext, group, state, param, grad, update, queue):
        # adam_wd is not forwarded, as in step() above
        return ext.adan_release(param, grad, state["exp_avg"], state["exp_avg_diff"], state["exp_avg_sq"], state["prev_grad"],
                         state["kahan_comp"], state["step"], group["lr"], group["beta1"], group["beta2"], group["beta3"],
                         group["weight_decay"], group["eps"], group["decouple_lr"], group["max_lr"], False,
                         bool(group["kahan_sum"]), update, queue)


class SGD(OptimiOptimizer):
    """SGD optimizer. Optionally with momentum and decoupled weight decay.

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        momentum: Momentum factor. Gradient moving average coefficient if `dampening` is True
            (default: 0)
        weight_decay: Weight decay coefficient. If `decouple_wd` and `decouple_lr` are False,
            applies L2 penalty (default: 0)
        dampening: Use dampening for momentum update (default: False)
        decouple_wd: Apply decoupled weight decay instead of L2 penalty (default: False)
        decouple_lr: Apply fully decoupled weight decay instead of L2 penalty (default: False)
        max_lr: Maximum scheduled learning rate. Set if `lr` is not the maximum scheduled learning
            rate and `decouple_lr` is True (default: None)
        torch_init: Initialize momentum buffer with first gradient instead of zeroes. Enable to
            match PyTorch SGD when using dampening (default: False)
        kahan_sum, foreach, triton, gradient_release: as `Adam`
    """

    _has_step = False

    _release_kind = "KIND_SGD"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        momentum: float = 0,
        weight_decay: float = 0,
        dampening: bool = False,
        decouple_wd: bool = False,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        torch_init: bool = False,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        if not 0.0 <= momentum < 1.0:
            raise ValueError(f"Invalid momentum: {momentum=}")
        defaults = dict(lr=lr, momentum=momentum, weight_decay=weight_decay, dampening=dampening,
                        decouple_wd=decouple_wd, decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum,
                        torch_init=torch_init, foreach=foreach, triton=triton, gradient_release=gradient_release,
                        setup=False)
        super().__init__(params, defaults)

    def _extra_state(self, group, state, param):
        # the momentum buffer: first gradient (torch's convention, after L2 decay), zeros, or absent
        # (optimi/sgd.py:97-107)
        if group["dampening"] and group["torch_init"]:
            state["exp_avg"] = param.grad.detach().clone()
            if group["weight_decay"] != 0 and not group["decouple_lr"] and not group["decouple_wd"]:
                # exp_avg.add_(param, alpha=wd) as ATen's CPU kernel computes it, which defines the
                # results: alpha narrowed to the tensor dtype, one fused multiply-add, one rounding
                # (float64 holds the product and the sum of two narrow floats exactly)
                alpha = float(torch.tensor(group["weight_decay"], dtype=param.dtype))
                fused = state["exp_avg"].double().add_(param.double(), alpha=alpha)
                state["exp_avg"] = fused.float().to(param.dtype)
        elif group["momentum"] != 0:
            state["exp_avg"] = torch.zeros_like(param, memory_format=torch.preserve_format)
        elif group["triton"]:
            state["exp_avg"] = torch.zeros(1, dtype=param.dtype, device=param.device)
        else:
            state["exp_avg"] = None

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        F.sgd(params, grads, _col(states, "exp_avg"), _col(states, "kahan_comp"), lr=group["lr"],
              momentum=group["momentum"], weight_decay=group["weight_decay"], dampening=group["dampening"],
              decouple_wd=group["decouple_wd"], decouple_lr=group["decouple_lr"], max_lr=group["max_lr"],
              kahan_sum=group["kahan_sum"], foreach=False, triton=True, gradient_release=gradient_release,
              optimizer_accumulation=accumulate, _groups=self._workspaces(group), _resident=self._lists_are_resident())

    def _release_call(self, ext, group, state, param, grad, update, queue):
        return ext.sgd_release(param, grad, state["exp_avg"], state["kahan_comp"], group["lr"], group["momentum"],
                        group["weight_decay"], group["dampening"], group["decouple_wd"], group["decouple_lr"],
                        group["max_lr"], bool(group["kahan_sum"]), update, queue)


class RAdam(OptimiOptimizer):
    """Rectified Adam optimizer. Optionally with decoupled weight decay.

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        betas: Coefficients for gradient and squared gradient moving averages (default: (0.9, 0.99))
        weight_decay: Weight decay coefficient. If `decouple_wd` and `decouple_lr` are False,
            applies L2 penalty (default: 0)
        eps: Added to denominator to improve numerical stability (default: 1e-6)
        decouple_wd: Apply decoupled weight decay instead of L2 penalty (default: False)
        decouple_lr, max_lr, kahan_sum, foreach, triton, gradient_release: as `Adam`
    """

    _moment_keys = ("exp_avg", "exp_avg_sq")

    _release_kind = "KIND_RADAM"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 0,
        eps: float = 1e-6,
        decouple_wd: bool = False,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        _check_betas(betas)
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon: {eps=}")
        defaults = dict(lr=lr, beta1=betas[0], beta2=betas[1], eps=eps, weight_decay=weight_decay,
                        decouple_wd=decouple_wd, decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum,
                        foreach=foreach, triton=triton, gradient_release=gradient_release, setup=False)
        super().__init__(params, defaults)

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        F.radam(params, grads, _col(states, "exp_avg"), _col(states, "exp_avg_sq"), _col(states, "kahan_comp"),
                lr=group["lr"], beta1=group["beta1"], beta2=group["beta2"], weight_decay=group["weight_decay"],
                eps=group["eps"], step=step, decouple_wd=group["decouple_wd"], decouple_lr=group["decouple_lr"],
                max_lr=group["max_lr"], kahan_sum=group["kahan_sum"], foreach=False, triton=True,
                gradient_release=gradient_release, optimizer_accumulation=accumulate, _groups=self._workspaces(group), _resident=self._lists_are_resident())

    def _release_call(self, ext, group, state, param, grad, update, queue):
        return ext.ranger_release(param, grad, state["exp_avg"], state["exp_avg_sq"], None, state["kahan_comp"], state["step"],
                           group["lr"], group["beta1"], group["beta2"], group["weight_decay"], group["eps"], 1, 0.0,
                           group["decouple_wd"], group["decouple_lr"], group["max_lr"], bool(group["kahan_sum"]), update, queue)


class Ranger(OptimiOptimizer):
    """Ranger optimizer. RAdam with Lookahead.

    Args:
        params: Iterable of parameters to optimize or dicts defining parameter groups
        lr: Learning rate
        betas: Coefficients for gradient and squared gradient moving averages (default: (0.9, 0.99))
        weight_decay: Weight decay coefficient. If `decouple_wd` and `decouple_lr` are False,
            applies L2 penalty (default: 0)
        eps: Added to denominator to improve numerical stability (default: 1e-6)
        k: Lookahead synchronization period (default: 6)
        alpha: Lookahead weight interpolation coefficient (default: 0.5)
        decouple_wd: Apply decoupled weight decay instead of L2 penalty (default: True)
        decouple_lr, max_lr, kahan_sum, foreach, triton, gradient_release: as `Adam`
    """

    _moment_keys = ("exp_avg", "exp_avg_sq")

    _release_kind = "KIND_RANGER"

    def __init__(
        self,
        params: Iterable[Tensor] | Iterable[dict],
        lr: float,
        betas: tuple[float, float] = (0.9, 0.99),
        weight_decay: float = 0,
        eps: float = 1e-6,
        k: int = 6,
        alpha: float = 0.5,
        decouple_wd: bool = True,
        decouple_lr: bool = False,
        max_lr: float | None = None,
        kahan_sum: bool | None = None,
        foreach: bool | None = None,
        triton: bool | None = None,
        gradient_release: bool = False,
    ):
        _check_betas(betas)
        if not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon: {eps=}")
        defaults = dict(lr=lr, beta1=betas[0], beta2=betas[1], eps=eps, weight_decay=weight_decay, k=k, alpha=alpha,
                        decouple_wd=decouple_wd, decouple_lr=decouple_lr, max_lr=max_lr, kahan_sum=kahan_sum,
                        foreach=foreach, triton=triton, gradient_release=gradient_release, setup=False)
        super().__init__(params, defaults)

    def _extra_state(self, group, state, param):
        state["la_param"] = param.data.clone()  # the slow weights start at the parameters (optimi/ranger.py:142)

    def _functional(self, group, params, grads, states, step, gradient_release, accumulate):
        F.ranger(params, grads, _col(states, "exp_avg"), _col(states, "exp_avg_sq"), _col(states, "la_param"),
                 _col(states, "kahan_comp"), lr=group["lr"], beta1=group["beta1"], beta2=group["beta2"],
                 weight_decay=group["weight_decay"], eps=group["eps"], k=group["k"], alpha=group["alpha"], step=step,
                 decouple_wd=group["decouple_wd"], decouple_lr=group["decouple_lr"], max_lr=group["max_lr"],
                 kahan_sum=group["kahan_sum"], foreach=False, triton=True, gradient_release=gradient_release,
                 optimizer_accumulation=accumulate, _groups=self._workspaces(group), _resident=self._lists_are_resident())

    def _release_call(self, ext, group, state, param, grad, update, queue):
        return ext.ranger_release(param, grad, state["exp_avg"], state["exp_avg_sq"], state["la_param"], state["kahan_comp"],
                           state["step"], group["lr"], group["beta1"], group["beta2"], group["weight_decay"],
                           group["eps"], group["k"], group["alpha"], group["decouple_wd"], group["decouple_lr"],
                           group["max_lr"], bool(group["kahan_sum"]), update, queue)
