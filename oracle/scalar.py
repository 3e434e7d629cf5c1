"""ctypes front end of the scalar C emulator (oracle/scalar_ref.c).

TEST INFRASTRUCTURE ONLY – see ``oracle/__init__.py``.

``ScalarRun`` has the ``step`` / ``step_param`` interface of
``oracle.forloop.ForLoopRun`` but forms the per-step scalars itself and hands
raw CPU buffers to the C functions, so the two oracles share no arithmetic.
"""

from __future__ import annotations

import ctypes as C
import math
import os
import subprocess

import torch

from .forloop import ForLoopRun

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboptimi_ref.so")

F32, BF16, F16 = 0, 1, 2
KAHAN, UPDATE, DECOUPLE_WD, ADAM_WD, DECOUPLE_LR, DAMPENING, RECTIFY, LOOKAHEAD = 1, 2, 4, 8, 16, 32, 64, 128

_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-B", "liboptimi_ref.so"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        d, p, i64, i = C.c_double, C.c_void_p, C.c_int64, C.c_int
        L.optimi_ref_adam.argtypes = [p, p, p, p, p, i64, i, d, d, d, d, d, d, i]
        L.optimi_ref_adam.restype = None
        L.optimi_ref_lion.argtypes = [p, p, p, p, i64, i, d, d, d, d, i]
        L.optimi_ref_lion.restype = None
        L.optimi_ref_stableadamw.argtypes = [p, p, p, p, p, i64, i, d, d, d, d, d, d, d, i]
        L.optimi_ref_stableadamw.restype = d
        L.optimi_ref_adan.argtypes = [p, p, p, p, p, p, p, i64, i, d, d, d, d, d, d, d, d, i]
        L.optimi_ref_adan.restype = None
        L.optimi_ref_round.argtypes = [C.c_float, i]
        L.optimi_ref_round.restype = C.c_float
        L.optimi_ref_sgd.argtypes = [p, p, p, p, i64, i, d, d, d, i]
        L.optimi_ref_sgd.restype = None
        L.optimi_ref_ranger.argtypes = [p, p, p, p, p, p, i64, i, d, d, d, d, d, d, d, d, i]
        L.optimi_ref_ranger.restype = None
        _lib = L
    return _lib


def _dt(t: torch.Tensor) -> int:
    assert t.device.type == "cpu" and t.is_contiguous()
    return {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}[t.dtype]


def _ptr(t):
    return None if t is None else t.data_ptr()


def _beta_hat(beta: float, t: int) -> float:
    """(beta^t - beta)/(beta^t - 1)   optimi/utils.py:31-36"""
    bt = beta**t
    return (bt - beta) / (bt - 1)


def step_scalars(name: str, h: dict, t: int | None, kahan_sum: bool, accumulate: bool, functional: bool = False):
    """The scalar arguments of one step, in the order the C entry points take them after
    ``dtype``: formed from the raw hyper-parameters ``h`` the way the reference's functional
    forms do (optimi/adam.py:260-273, lion.py:226-235, stableadamw.py:326-332, adan.py:289-309).
    ``t`` is the already advanced step count (None for Lion).  ``functional``: the caller is the
    functional form itself, not a class, so Adan's ``adam_wd`` is honoured (adan.py:300-309); the
    classes never forward it (adan.py:181-203)."""
    lr, wd = h["lr"], h.get("weight_decay", 0.0)
    flags = (KAHAN if kahan_sum else 0) | (0 if accumulate else UPDATE)
    ratio = lr / h["max_lr"] if h.get("decouple_lr") else lr  # lr, or lr/max_lr when fully decoupled
    if name in ("adam", "adamw"):
        b1, b2 = h.get("betas", (0.9, 0.99))
        b1h, b2h = _beta_hat(b1, t), _beta_hat(b2, t)
        decoupled = name == "adamw" or h.get("decouple_wd", False) or h.get("decouple_lr", False)
        w = 1 - ratio * wd if (wd != 0 and decoupled) else wd
        return (lr, 1 - b1h, b2h, 1 - b2h, w, h["eps"], flags | (DECOUPLE_WD if decoupled else 0))
    if name == "lion":
        b1, b2 = h.get("betas", (0.9, 0.99))
        w = 1 - ratio * wd if wd != 0 else 0.0
        return (lr, 1 - b1, 1 - b2, w, flags)
    if name == "stableadamw":
        b1, b2 = h.get("betas", (0.9, 0.99))
        b1h, b2h = _beta_hat(b1, t), _beta_hat(b2, t)
        dl = bool(h.get("decouple_lr"))
        return (lr, 1 - b1h, b2h, 1 - b2h, wd, h["eps"], h["max_lr"] if dl else 0.0, flags | (DECOUPLE_LR if dl else 0))
    if name == "adan":
        b1, b2, b3 = h.get("betas", (0.98, 0.92, 0.99))
        b1h, b2h, b3h = _beta_hat(b1, t), _beta_hat(b2, t), _beta_hat(b3, t)
        adam_wd = bool(functional and h.get("adam_wd"))  # the class path is always Adan-style (adan.py:181-203)
        w = 0.0
        if wd != 0:
            w = 1 - ratio * wd if adam_wd else 1 + ratio * wd
        return (lr, 1 - b1h, b2, 1 - b2h, b3h, 1 - b3h, h["eps"], w, flags | (ADAM_WD if adam_wd else 0))
    if name == "sgd":
        decoupled = bool(h.get("decouple_wd") or h.get("decouple_lr"))
        w = 1 - ratio * wd if (wd != 0 and decoupled) else wd
        return (lr, h.get("momentum", 0.0), w,
                flags | (DECOUPLE_WD if decoupled else 0) | (DAMPENING if h.get("dampening") else 0))
    if name in ("radam", "ranger"):
        b1, b2 = h.get("betas", (0.9, 0.99))
        b1h, b2h = _beta_hat(b1, t), _beta_hat(b2, t)
        decoupled = bool(h.get("decouple_wd") or h.get("decouple_lr"))
        w = 1 - ratio * wd if (wd != 0 and decoupled) else wd
        rect = rectification(b2, t)
        f = flags | (DECOUPLE_WD if decoupled else 0) | (RECTIFY if rect is not None else 0)
        if name == "ranger" and t % h.get("k", 6) == 0:
            f |= LOOKAHEAD
        head = (lr, 1 - b1h, b2h, 1 - b2h, w, h["eps"], rect if rect is not None else 0.0)
        return head + ((h.get("alpha", 0.5), f) if name == "ranger" else (f,))
    raise ValueError(name)


def rectification(beta2: float, t: int):
    """RAdam's variance rectification term or None  (optimi/radam.py:269-277)."""
    rho_inf = 2 / (1 - beta2) - 1
    rho = rho_inf - 2 * t * (beta2**t) / (1 - beta2**t)
    if rho > 5:
        return math.sqrt(((rho - 4) * (rho - 2) * rho_inf) / ((rho_inf - 4) * (rho_inf - 2) * rho))
    return None


# state buffers each C entry point takes between ``grad`` and ``kahan_comp``
STATE_ORDER = {
    "adam": ("exp_avg", "exp_avg_sq"),
    "adamw": ("exp_avg", "exp_avg_sq"),
    "lion": ("exp_avg",),
    "stableadamw": ("exp_avg", "exp_avg_sq"),
    "adan": ("exp_avg", "exp_avg_diff", "exp_avg_sq", "prev_grad"),
    "sgd": ("exp_avg",),
    "radam": ("exp_avg", "exp_avg_sq"),
    "ranger": ("exp_avg", "exp_avg_sq", "la_param"),
}


class ScalarRun(ForLoopRun):
    """Same state handling as ``ForLoopRun``; the arithmetic is the C emulator's."""

    def _call(self, idxs, grads, step, accumulate):
        L = lib()
        t = None
        if self.name not in ("lion", "sgd"):
            step.add_(1)
            t = int(step.item())
        scalars = step_scalars(self.name, self.hyper, t, self.kahan_sum, accumulate, self.functional)
        fn = {"adam": L.optimi_ref_adam, "adamw": L.optimi_ref_adam, "lion": L.optimi_ref_lion,
              "stableadamw": L.optimi_ref_stableadamw, "adan": L.optimi_ref_adan, "sgd": L.optimi_ref_sgd,
              "radam": L.optimi_ref_ranger, "ranger": L.optimi_ref_ranger}[self.name]
        for i, g in zip(idxs, grads):
            st = self._ensure_state(i, g)
            p = self.params[i]
            bufs = [_ptr(st[k]) for k in STATE_ORDER[self.name]]
            args = scalars
            if self.name == "radam":  # the C function serves RAdam and Ranger: no slow weights, no alpha
                bufs.append(None)
                args = scalars[:-1] + (0.0, scalars[-1])
            fn(_ptr(p), _ptr(g), *bufs, _ptr(st["kahan_comp"]), p.numel(), _dt(p), *args)
