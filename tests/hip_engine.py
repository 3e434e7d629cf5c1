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

    def __init__(self, name, params, *, multi=True, cold=False, mixed=False, **kw):
        super().__init__(name, params, **kw)
        self.multi = multi
        self.cold = cold  # pass OPTIMI_COLD to the whole-list entry points
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
            if self.cold:
                scalars = scalars[:-1] + (scalars[-1] | cabi.COLD,)
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
