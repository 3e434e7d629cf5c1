"""Drives the HIP library through its C ABI with the ``step`` / ``step_param`` interface of
``oracle.forloop.ForLoopRun``, so the same replay code feeds the oracle and the kernels.

torch only provides device memory and the stream here: every launch goes through
``optimi_amd.cabi`` (ctypes on ``liboptimi_hip.so``).  Step scalars come from
``oracle.scalar.step_scalars`` – the prologue the golden fixtures pin.
"""

from __future__ import annotations

import ctypes as C

import torch

from optimi_amd import cabi
from oracle.forloop import ForLoopRun
from oracle.scalar import STATE_ORDER, step_scalars

DT = {torch.float32: cabi.F32, torch.bfloat16: cabi.BF16, torch.float16: cabi.F16}


def _addr(t):
    return None if t is None else t.data_ptr()


class HipRun(ForLoopRun):
    """``multi=True``: whole-list entry points (one launch); False: per-tensor entry points.
    A list whose tensors differ in dtype goes through the ``_multi_mixed`` entry points;
    ``mixed=True`` sends a list of one dtype through them as well."""

    def __init__(self, name, params, *, multi=True, resident=False, mixed=False, **kw):
        super().__init__(name, params, **kw)
        self.multi = multi
        self.resident = resident  # pass OPTIMI_RESIDENT to the whole-list entry points
        self.mixed = mixed
        self.group = cabi.Group()
        self.entry = "adam" if name == "adamw" else name

    def _ensure_state(self, i, grad):
        """A state that starts from arithmetic (SGD's ``torch_init`` momentum buffer) is built by the
        oracle's own code on CPU copies and moved to the device, so that it starts from the CPU result;
        every other state is zeros or a copy and is created on the device."""
        arithmetic = self.name == "sgd" and self.hyper.get("dampening") and self.hyper.get("torch_init")
        if self.state[i] is not None or not arithmetic:
            return super()._ensure_state(i, grad)
        p_dev = self.params[i]
        self.params[i] = p_dev.detach().cpu()
        try:
            st = super()._ensure_state(i, grad.detach().cpu())
        finally:
            self.params[i] = p_dev
        for k, v in st.items():
            if torch.is_tensor(v) and k != "step":
                st[k] = v.to(p_dev.device)
        return st

    def _stream(self):
        return torch.cuda.current_stream().cuda_stream

    def _call(self, idxs, grads, step, accumulate):
        L = cabi.lib()
        t = None
        if self.name not in ("lion", "sgd"):
            step.add_(1)
            t = int(step.item())
        scalars = step_scalars(self.name, self.hyper, t, self.kahan_sum, accumulate, self.functional)
        sts = [self._ensure_state(i, g) for i, g in zip(idxs, grads)]
        ps = [self.params[i] for i in idxs]
        if not ps:
            return
        dt = DT[ps[0].dtype]
        if self.multi and not self.gradient_release:
            if self.resident:
                scalars = scalars[:-1] + (scalars[-1] | cabi.RESIDENT,)
            cols = [cabi.ptr_array(_addr(p) for p in ps), cabi.ptr_array(_addr(g) for g in grads)]
            cols += [cabi.ptr_array(_addr(s[k]) for s in sts) for k in STATE_ORDER[self.name]]
            cols.append(cabi.ptr_array(_addr(s["kahan_comp"]) for s in sts))
            if self.mixed or len({p.dtype for p in ps}) > 1:
                fn = getattr(L, f"optimi_hip_{self.entry}_multi_mixed")
                dt = (C.c_int * len(ps))(*[DT[p.dtype] for p in ps])
            else:
                fn = getattr(L, f"optimi_hip_{self.entry}_multi")
            rc = fn(self.group.handle, len(ps), *cols, cabi.i64_array(p.numel() for p in ps), dt, *scalars, self._stream())
            cabi.check(rc, fn.__name__)
        else:
            fn = getattr(L, f"optimi_hip_{self.entry}_single")
            lead = (self.group.handle,) if self.entry == "stableadamw" else ()
            for p, g, s in zip(ps, grads, sts):
                bufs = [_addr(s[k]) for k in STATE_ORDER[self.name]]
                rc = fn(*lead, _addr(p), _addr(g), *bufs, _addr(s["kahan_comp"]), p.numel(), DT[p.dtype], *scalars, self._stream())
                cabi.check(rc, fn.__name__)


class FunctionalRun(HipRun):
    """The product's public functional forms, ``optimi_amd.adam`` ... ``optimi_amd.ranger``, called
    the way a direct caller of the reference's functional API calls them: lists of tensors for a
    whole-list step, bare tensors with ``gradient_release=True`` for a per-tensor step, raw
    hyper-parameters, the int32 CPU step counter, no launch workspace of the caller's."""

    def _call(self, idxs, grads, step, accumulate):
        ForLoopRun._call(self, idxs, grads, step, accumulate)

    def _invoke(self, form, columns, kwargs):
        import optimi_amd

        if self.gradient_release:  # the reference's hook hands over the tensors themselves
            assert all(len(c) == 1 for c in columns)
            columns = [c[0] for c in columns]
        getattr(optimi_amd, form)(*columns, triton=True, gradient_release=self.gradient_release, **kwargs)


class PlainHipRun:
    """The same C-ABI driver with nothing borrowed from ``oracle/``: states are made with plain
    ``torch.zeros_like`` / ``-grad`` / ``clone`` on the device, and the step scalars are formed here
    from the raw hyper-parameters with the product's own ``optimi_amd.utils.debias_beta``, following
    the reference's functional prologues line by line (optimi/adam.py:260-273, lion.py:226-235,
    stableadamw.py:326-332, adan.py:289-309, sgd.py:233-245, radam.py:262-284, ranger.py:281-305).
    An error shared by the oracle's driver (``ForLoopRun._ensure_state``, ``oracle.scalar.step_scalars``)
    and ``HipRun``, which inherits it, would pass unseen there; it cannot here."""

    DEFAULTS = {
        "adam": dict(betas=(0.9, 0.99), weight_decay=0.0, eps=1e-6, decouple_wd=False),
        "adamw": dict(betas=(0.9, 0.99), weight_decay=1e-2, eps=1e-6, decouple_wd=True),
        "lion": dict(betas=(0.9, 0.99), weight_decay=0.0),
        "stableadamw": dict(betas=(0.9, 0.99), weight_decay=1e-2, eps=1e-6),
        "adan": dict(betas=(0.98, 0.92, 0.99), weight_decay=2e-2, eps=1e-6, kahan_sum=False),
        "sgd": dict(momentum=0.0, weight_decay=0.0, dampening=False, decouple_wd=False, torch_init=False),
        "radam": dict(betas=(0.9, 0.99), weight_decay=0.0, eps=1e-6, decouple_wd=False),
        "ranger": dict(betas=(0.9, 0.99), weight_decay=0.0, eps=1e-6, k=6, alpha=0.5, decouple_wd=True),
    }
    STATES = {"adam": ("exp_avg", "exp_avg_sq"), "adamw": ("exp_avg", "exp_avg_sq"), "lion": ("exp_avg",),
              "stableadamw": ("exp_avg", "exp_avg_sq"), "adan": ("exp_avg", "exp_avg_diff", "exp_avg_sq", "prev_grad"),
              "sgd": ("exp_avg",), "radam": ("exp_avg", "exp_avg_sq"), "ranger": ("exp_avg", "exp_avg_sq", "la_param")}

    def __init__(self, name, params, *, multi=True, gradient_release=False, functional=False, **hyper):
        self.name, self.params, self.multi = name, list(params), multi
        self.gradient_release, self.functional = gradient_release, functional
        h = {**self.DEFAULTS[name], **hyper}
        if h.get("decouple_lr") and h.get("max_lr") is None:
            h["max_lr"] = h["lr"]
        ks = h.pop("kahan_sum", None)
        low = (torch.bfloat16, torch.float16)
        self.kahan = [(ks or ks is None) and p.dtype in low for p in self.params]
        self.kahan_sum = any(self.kahan) or bool(ks)
        self.h = h
        self.state = [None] * len(self.params)
        self.group_step = 0
        self.optimizer_accumulation = False
        self.group = cabi.Group()
        self.entry = "adam" if name == "adamw" else name

    def _state(self, i, grad):
        if self.state[i] is None:
            p, h = self.params[i], self.h
            st = {"exp_avg": torch.zeros_like(p)}
            if self.name == "sgd":
                if h["dampening"] and h["torch_init"]:
                    st["exp_avg"] = grad.clone()
                    if h["weight_decay"] != 0 and not h.get("decouple_lr") and not h["decouple_wd"]:
                        # g + wd*p with wd narrowed to the tensor dtype, fused, rounded once (what ATen's CPU add_ gives)
                        alpha = float(torch.tensor(h["weight_decay"], dtype=p.dtype))
                        st["exp_avg"] = (grad.double() + alpha * p.double()).float().to(p.dtype)
                elif h["momentum"] == 0:
                    st["exp_avg"] = None
            if "exp_avg_sq" in self.STATES[self.name]:
                st["exp_avg_sq"] = torch.zeros_like(p)
            if self.name == "ranger":
                st["la_param"] = p.clone()
            if self.name == "adan":
                st["exp_avg_diff"] = torch.zeros_like(p)
                st["prev_grad"] = -grad
            st["kahan_comp"] = torch.zeros_like(p) if self.kahan[i] else None
            st["step"] = 0
            self.state[i] = st
        return self.state[i]

    def _scalars(self, t, accumulate):
        from optimi_amd.functional import _rectification
        from optimi_amd.utils import debias_beta

        h, name = self.h, self.name
        lr, wd = h["lr"], h["weight_decay"]
        flags = (cabi.KAHAN if self.kahan_sum else 0) | (0 if accumulate else cabi.UPDATE)
        decouple_lr = bool(h.get("decouple_lr"))

        def factor(decoupled):  # 1 - lr*wd, 1 - (lr/max_lr)*wd, or the raw coefficient for L2
            if wd == 0:
                return 0.0
            if decouple_lr:
                return 1 - (lr / h["max_lr"]) * wd
            return 1 - lr * wd if decoupled else wd

        if name in ("adam", "adamw", "radam", "ranger"):
            b1, b2 = h["betas"]
            b1h, b2h = debias_beta(b1, t), debias_beta(b2, t)
            decoupled = bool(h["decouple_wd"]) or decouple_lr
            flags |= cabi.DECOUPLE_WD if decoupled else 0
            head = (lr, 1 - b1h, b2h, 1 - b2h, factor(decoupled), h["eps"])
            if name in ("adam", "adamw"):
                return head + (flags,)
            rect = _rectification(b2, t)
            flags |= cabi.RECTIFY if rect is not None else 0
            tail = (rect if rect is not None else 0.0,)
            if name == "ranger":
                flags |= cabi.LOOKAHEAD if t % h["k"] == 0 else 0
                tail += (h["alpha"],)
            return head + tail + (flags,)
        if name == "lion":
            b1, b2 = h["betas"]
            return (lr, 1 - b1, 1 - b2, factor(True), flags)
        if name == "stableadamw":
            b1, b2 = h["betas"]
            b1h, b2h = debias_beta(b1, t), debias_beta(b2, t)
            return (lr, 1 - b1h, b2h, 1 - b2h, wd, h["eps"], h["max_lr"] if decouple_lr else 0.0,
                    flags | (cabi.DECOUPLE_LR if decouple_lr else 0))
        if name == "adan":
            b1, b2, b3 = h["betas"]
            b1h, b2h, b3h = debias_beta(b1, t), debias_beta(b2, t), debias_beta(b3, t)
            # only a direct caller of the functional form reaches Adam-style decay (optimi/adan.py:181-203)
            adam_wd = bool(self.functional and h.get("adam_wd"))
            w = 0.0
            if wd != 0:
                w = (lr / h["max_lr"]) * wd if decouple_lr else lr * wd
                w = 1 - w if adam_wd else 1 + w
            return (lr, 1 - b1h, b2, 1 - b2h, b3h, 1 - b3h, h["eps"], w, flags | (cabi.ADAM_WD if adam_wd else 0))
        if name == "sgd":
            decoupled = bool(h["decouple_wd"]) or decouple_lr
            return (lr, h["momentum"], factor(decoupled),
                    flags | (cabi.DECOUPLE_WD if decoupled else 0) | (cabi.DAMPENING if h["dampening"] else 0))
        raise ValueError(name)

    def _launch(self, idxs, grads, t, accumulate):
        if not idxs:
            return
        L = cabi.lib()
        scalars = self._scalars(t, accumulate)
        sts = [self._state(i, g) for i, g in zip(idxs, grads)]
        ps = [self.params[i] for i in idxs]
        stream = torch.cuda.current_stream().cuda_stream
        if self.multi and not self.gradient_release:
            cols = [cabi.ptr_array(_addr(p) for p in ps), cabi.ptr_array(_addr(g) for g in grads)]
            cols += [cabi.ptr_array(_addr(s[k]) for s in sts) for k in self.STATES[self.name]]
            cols.append(cabi.ptr_array(_addr(s["kahan_comp"]) for s in sts))
            if len({p.dtype for p in ps}) > 1:
                fn = getattr(L, f"optimi_hip_{self.entry}_multi_mixed")
                dt = (C.c_int * len(ps))(*[DT[p.dtype] for p in ps])
            else:
                fn = getattr(L, f"optimi_hip_{self.entry}_multi")
                dt = DT[ps[0].dtype]
            cabi.check(fn(self.group.handle, len(ps), *cols, cabi.i64_array(p.numel() for p in ps), dt, *scalars, stream),
                       fn.__name__)
        else:
            fn = getattr(L, f"optimi_hip_{self.entry}_single")
            lead = (self.group.handle,) if self.entry == "stableadamw" else ()
            for p, g, s in zip(ps, grads, sts):
                bufs = [_addr(s[k]) for k in self.STATES[self.name]]
                cabi.check(fn(*lead, _addr(p), _addr(g), *bufs, _addr(s["kahan_comp"]), p.numel(), DT[p.dtype], *scalars, stream),
                           fn.__name__)

    def step(self, grads):
        idxs = [i for i, g in enumerate(grads) if g is not None]
        gs = [grads[i] for i in idxs]
        for i, g in zip(idxs, gs):
            self._state(i, g)
        self.group_step += 1
        self._launch(idxs, gs, self.group_step, False)

    def step_param(self, i, grad):
        st = self._state(i, grad)
        st["step"] += 1
        self._launch([i], [grad], st["step"], self.optimizer_accumulation)
