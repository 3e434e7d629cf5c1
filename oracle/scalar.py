"""ctypes front end of the scalar C emulator (oracle/scalar_ref.c).

TEST INFRASTRUCTURE ONLY – see ``oracle/__init__.py``.

``ScalarRun`` has the ``step`` / ``step_param`` interface of
``oracle.forloop.ForLoopRun`` but forms the per-step scalars itself and hands
raw CPU buffers to the C functions, so the two oracles share no arithmetic.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import torch

from .forloop import ForLoopRun

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboptimi_ref.so")

F32, BF16 = 0, 1
KAHAN, UPDATE, DECOUPLE_WD, ADAM_WD, DECOUPLE_LR = 1, 2, 4, 8, 16

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
        _lib = L
    return _lib


def _dt(t: torch.Tensor) -> int:
    assert t.device.type == "cpu" and t.is_contiguous()
    return {torch.float32: F32, torch.bfloat16: BF16}[t.dtype]


def _ptr(t):
    return None if t is None else t.data_ptr()


def _beta_hat(beta: float, t: int) -> float:
    """(beta^t - beta)/(beta^t - 1)   optimi/utils.py:31-36"""
    bt = beta**t
    return (bt - beta) / (bt - 1)


class ScalarRun(ForLoopRun):
    """Same state handling as ``ForLoopRun``; the arithmetic is the C emulator's."""

    def _call(self, idxs, grads, step, accumulate):
        L = lib()
        h = self.hyper
        lr, wd = h["lr"], h.get("weight_decay", 0.0)
        flags = (KAHAN if self.kahan_sum else 0) | (0 if accumulate else UPDATE)
        if self.name != "lion":
            step.add_(1)
            t = int(step.item())
        ratio = lr / h["max_lr"] if h.get("decouple_lr") else lr  # lr, or lr/max_lr when fully decoupled
        for i, g in zip(idxs, grads):
            st = self._ensure_state(i, g)
            p = self.params[i]
            n, dt = p.numel(), _dt(p)
            if self.name in ("adam", "adamw"):
                b1, b2 = h.get("betas", (0.9, 0.99))
                b1h, b2h = _beta_hat(b1, t), _beta_hat(b2, t)
                decoupled = self.name == "adamw" or h.get("decouple_wd", False) or h.get("decouple_lr", False)
                w = wd
                if wd != 0 and decoupled:  # adam.py:269-273
                    w = 1 - ratio * wd
                L.optimi_ref_adam(_ptr(p), _ptr(g), _ptr(st["exp_avg"]), _ptr(st["exp_avg_sq"]), _ptr(st["kahan_comp"]),
                                  n, dt, lr, 1 - b1h, b2h, 1 - b2h, w, h["eps"],
                                  flags | (DECOUPLE_WD if decoupled else 0))
            elif self.name == "lion":
                b1, b2 = h.get("betas", (0.9, 0.99))
                w = 1 - ratio * wd if wd != 0 else 0.0  # lion.py:226-231
                L.optimi_ref_lion(_ptr(p), _ptr(g), _ptr(st["exp_avg"]), _ptr(st["kahan_comp"]), n, dt, lr, 1 - b1,
                                  1 - b2, w, flags)
            elif self.name == "stableadamw":
                b1, b2 = h.get("betas", (0.9, 0.99))
                b1h, b2h = _beta_hat(b1, t), _beta_hat(b2, t)
                dl = bool(h.get("decouple_lr"))
                L.optimi_ref_stableadamw(_ptr(p), _ptr(g), _ptr(st["exp_avg"]), _ptr(st["exp_avg_sq"]),
                                         _ptr(st["kahan_comp"]), n, dt, lr, 1 - b1h, b2h, 1 - b2h, wd, h["eps"],
                                         h["max_lr"] if dl else 0.0, flags | (DECOUPLE_LR if dl else 0))
            elif self.name == "adan":
                b1, b2, b3 = h.get("betas", (0.98, 0.92, 0.99))
                b1h, b2h, b3h = _beta_hat(b1, t), _beta_hat(b2, t), _beta_hat(b3, t)
                w = 1 + ratio * wd if wd != 0 else 0.0  # adan.py:300-309; the class path is always Adan-style
                L.optimi_ref_adan(_ptr(p), _ptr(g), _ptr(st["exp_avg"]), _ptr(st["exp_avg_diff"]),
                                  _ptr(st["exp_avg_sq"]), _ptr(st["prev_grad"]), _ptr(st["kahan_comp"]), n, dt, lr,
                                  1 - b1h, b2, 1 - b2h, b3h, 1 - b3h, h["eps"], w, flags)
            else:
                raise ValueError(self.name)
