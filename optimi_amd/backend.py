"""Loads the native pieces and fails loudly when they are missing.

``ext()`` returns the PyTorch-ROCm binding (``optimi_amd._C``), which itself links
``liboptimi_hip.so``.  There is no Python or CPU fallback: if the binding cannot be
imported, or a tensor is not on a HIP device, the caller gets an exception.
"""

from __future__ import annotations

import threading

import torch

_ext = None
_ext_error: Exception | None = None
_lock = threading.Lock()


def ext():
    global _ext, _ext_error
    if _ext is None:
        with _lock:
            if _ext is None:
                try:
                    from . import _C  # noqa: PLC0415
                except ImportError as err:  # pragma: no cover - depends on the build
                    _ext_error = err
                    raise ImportError(
                        "optimi_amd: the HIP extension is not built. Run `python -m optimi_amd.build` "
                        "(needs hipcc and PyTorch-ROCm); there is no fallback backend."
                    ) from err
                _ext = _C
    return _ext


_thread = threading.local()


def default_group(device: torch.device, dtype: torch.dtype, tag: str = ""):
    """A per-thread launch workspace for functional calls that bring none of their own; it goes
    when its thread does."""
    groups = _thread.__dict__.setdefault("groups", {})
    key = (device.type, device.index, dtype, tag)
    grp = groups.get(key)
    if grp is None:
        with torch.cuda.device(device):
            grp = ext().Group()
        groups[key] = grp
    return grp


SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


def check_supported(param: torch.Tensor):
    if not param.is_cuda:
        raise RuntimeError(
            f"optimi_amd runs on HIP devices only; got a parameter on {param.device}. "
            "There is no CPU path in this package."
        )
    if param.dtype not in SUPPORTED_DTYPES:
        raise NotImplementedError(f"optimi_amd: parameter dtype {param.dtype} is not implemented (float32, bfloat16 and float16 are)")


def like_param(param: torch.Tensor, other: torch.Tensor) -> torch.Tensor:
    """``other`` laid out like ``param`` (a copy only when strides differ)."""
    if other.stride() == param.stride():
        return other
    return torch.empty_like(param, memory_format=torch.preserve_format).copy_(other)
