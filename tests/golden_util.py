"""Loading and replaying the golden fixtures (tests/golden/*.npz).

A fixture holds the inputs the reference saw (initial params, the gradient of
every step) and what its for-loop path produced (params and states after
selected steps).  ``replay`` feeds the same inputs to any engine with the
small ``step`` / ``step_param`` interface of ``oracle.forloop.ForLoopRun`` and
returns the snapshots in the fixture's own key layout.
"""

from __future__ import annotations

import glob
import importlib.util
import os

import numpy as np
import torch

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN_DIR, "make_fixtures.py"))
_mk = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_mk)
CASES = _mk.CASES
SEEDS = _mk.SEEDS
make_inputs = _mk.make_inputs
case_dtypes = _mk.case_dtypes
STATE_KEYS = _mk.STATE_KEYS
N_TENSORS = len(_mk.SHAPES)

OPT_NAME = {"Adam": "adam", "AdamW": "adamw", "Lion": "lion", "StableAdamW": "stableadamw", "Adan": "adan",
            "SGD": "sgd", "RAdam": "radam", "Ranger": "ranger"}


def torch_tail(name: str, numel: int, dtype: torch.dtype | None = None) -> int:
    """How many trailing elements of a bf16 or fp16 tensor (``dtype``; by default the dtype of the
    case) of a fixture case to leave out when comparing
    against anything but torch itself.  ATen's CPU ``add_(other, alpha=...)`` fuses
    ``self + alpha*other`` in fp32 in its vector body but works in bf16 arithmetic (the product
    rounded on its own) in the scalar loop over the last ``numel % 32`` elements, so the
    reference's own output is not uniform there.  SGD (``p += -lr*m``), RAdam/Ranger before
    rectification, Ranger's Lookahead and L2 weight decay go through that op; the kernels and
    the C emulator follow the vector body everywhere."""
    low = CASES[name][2] in ("bfloat16", "float16") if dtype is None else dtype in (torch.bfloat16, torch.float16)
    uses_add_alpha = name.split("_")[0] in ("sgd", "radam", "ranger") or name.endswith("_l2")
    return numel % 32 if (low and uses_add_alpha) else 0


def case_names(functional: bool | None = None):
    """All fixture cases; ``functional`` False / True keeps only the cases written through the
    reference's classes / through its functional form."""
    names = sorted(n for n in CASES if functional is None or CASES[n][3].startswith("functional") == functional)
    have = {os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN_DIR, "*.npz"))}
    assert set(names) <= have, f"fixtures missing: {sorted(set(names) - have)}"
    return names


def from_np(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(a.copy())


def load(name: str) -> dict[str, torch.Tensor]:
    with np.load(os.path.join(GOLDEN_DIR, f"{name}.npz"), allow_pickle=False) as z:
        return {k: from_np(z[k]) for k in z.files}


def snap_steps(fx: dict) -> list[int]:
    return sorted({int(k.split(".")[1]) for k in fx if k.startswith("out.")})


def replay(name: str, fx: dict, make_engine, device="cpu") -> dict[str, torch.Tensor]:
    """``make_engine(opt_name, params, gradient_release=..., **kwargs)`` → engine."""
    cls_name, kwargs, _dtype, mode, n_steps = CASES[name]
    params = [fx[f"in.param.{i}"].clone().to(device) for i in range(N_TENSORS)]
    release = mode in ("release", "functional_release")
    # "functional" cases were written by the reference's functional form called directly
    extra = {"functional": True} if mode.startswith("functional") else {}
    eng = make_engine(OPT_NAME[cls_name], params, gradient_release=release, **extra, **kwargs)
    wanted = set(snap_steps(fx))
    out = {}
    for t in range(n_steps):
        grads = [fx[f"in.grad.{t}.{i}"].clone().to(device) for i in range(N_TENSORS)]
        if release:
            eng.optimizer_accumulation = (t + 1) % 4 != 0
            for i in reversed(range(N_TENSORS)):
                eng.step_param(i, grads[i])
        else:
            eng.step(grads)
        if (t + 1) in wanted:
            for i in range(N_TENSORS):
                out[f"out.{t + 1}.param.{i}"] = eng.params[i].detach().cpu().clone()
                for key in STATE_KEYS:
                    st = eng.state[i].get(key) if eng.state[i] is not None else None
                    if torch.is_tensor(st) and st.numel() == eng.params[i].numel():
                        out[f"out.{t + 1}.{key}.{i}"] = st.detach().cpu().clone()
    return out


# ----------------------------------------------------------------------------
# comparison helpers
# ----------------------------------------------------------------------------
def bf16_ordinal(t: torch.Tensor) -> torch.Tensor:
    """Maps bf16 (or fp16) values to integers so that adjacent representable values differ by 1."""
    bits = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    neg = bits >= 0x8000
    # every NaN maps to one ordinal: its sign and payload are not part of the result
    return torch.where(torch.isnan(t), torch.full_like(bits, 1 << 20), torch.where(neg, 0x8000 - bits, bits))


def bf16_ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return (bf16_ordinal(a) - bf16_ordinal(b)).abs()


def bf16_ulp_of(t: torch.Tensor) -> torch.Tensor:
    """Size of one ulp of ``t``'s dtype (bf16 or fp16) at each value of ``t`` (as fp32)."""
    if t.dtype == torch.float16:
        f = t.float().abs().clamp_min(2.0**-14)  # subnormals share the ulp of the smallest normal
        return torch.exp2(torch.floor(torch.log2(f)) - 10)
    f = t.float().abs().clamp_min(2.0**-126)
    return torch.exp2(torch.floor(torch.log2(f)) - 7)


def fp32_rel_err(a: torch.Tensor, b: torch.Tensor, floor: float) -> torch.Tensor:
    """|a-b| / max(|a|,|b|, floor)."""
    a, b = a.double(), b.double()
    return (a - b).abs() / torch.maximum(torch.maximum(a.abs(), b.abs()), torch.tensor(floor, dtype=torch.float64))


# worst fp32 disagreement seen in this run with no floor applied: optimizer -> {"param" | "state": (rel, ulps, abs)}
FP32_WORST: dict = {}


def note_fp32_error(name: str, key: str, got: torch.Tensor, want: torch.Tensor):
    a, b = got.detach().cpu().float().flatten(), want.detach().cpu().float().flatten()
    fin = torch.isfinite(a) & torch.isfinite(b)
    a, b = a[fin], b[fin]
    if a.numel() == 0:
        return
    diff = (a.double() - b.double()).abs()
    big = torch.maximum(a.abs(), b.abs()).double()
    rel = torch.where(big > 0, diff / big.clamp_min(1e-300), torch.zeros_like(diff))
    i = int(rel.argmax())
    ulp = torch.exp2(torch.floor(torch.log2(big[i].clamp_min(2.0**-126))) - 23)
    kind = "param" if (".param." in key or ".la_param." in key) else "state"
    slot = FP32_WORST.setdefault(name.split("_")[0], {})
    if float(rel[i]) > slot.get(kind, (-1.0,))[0]:
        slot[kind] = (float(rel[i]), float(diff[i] / ulp), float(diff[i]), f"{name} {key}")


def assert_bits_equal(got: torch.Tensor, want: torch.Tensor, what: str):
    a = got.detach().cpu().contiguous()
    b = want.detach().cpu().contiguous()
    view = torch.int16 if a.dtype in (torch.bfloat16, torch.float16) else torch.int32
    bad = (a.view(view) != b.view(view)) & ~(torch.isnan(a) & torch.isnan(b))  # a NaN's sign and payload are free
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} elements differ (first at {int(bad.flatten().nonzero()[0])})"


def assert_close_to_reference(got, want, what, *, param=None, is_param=False):
    """The north-star tolerance: bf16 within 1 ulp (a Kahan buffer within 1 ulp of its parameter),
    fp32 within rel 1e-6.  The fp32 comparison is |a-b| <= 1e-6 * max(|a|, |b|, floor): elements
    that cancel towards zero carry the rounding error of the terms that cancelled, so they are
    judged against the size of those terms - 1e-2 for parameters (the distance ten steps can move
    a parameter at lr 1e-3; i.e. |a-b| <= 1e-8 near zero) and the tensor's RMS for moment states."""
    got, want = got.detach().cpu(), want.detach().cpu()
    # overflow and 0/0 must happen in the same places with the same outcome (fp16 reaches both);
    # the tolerance below then applies to the finite elements
    wild = ~torch.isfinite(want)
    if bool(wild.any()) or not bool(torch.isfinite(got).all()):
        assert torch.equal(torch.isnan(got), torch.isnan(want)), f"{what}: NaN in different places"
        inf = torch.isinf(want)
        assert torch.equal(torch.isinf(got), inf) and torch.equal(got[inf], want[inf]), f"{what}: inf in different places"
        got, want = got.masked_fill(wild, 0), want.masked_fill(wild, 0)
        if param is not None:
            param = param.detach().cpu()
            got, want = got.masked_fill(~torch.isfinite(param), 0), want.masked_fill(~torch.isfinite(param), 0)
            param = param.masked_fill(~torch.isfinite(param), 1)
    if want.dtype in (torch.bfloat16, torch.float16):
        if param is not None:
            err = (got.float() - want.float()).abs() / bf16_ulp_of(param.detach().cpu())
            assert float(err.max()) <= 1.0, f"{what}: Kahan buffer off by {float(err.max()):.3f} parameter ulps"
        else:
            ulp = bf16_ulp_diff(got, want)
            assert int(ulp.max()) <= 1, f"{what}: {int((ulp > 1).sum())} elements beyond 1 ulp (max {int(ulp.max())})"
    else:
        floor = 1e-2 if is_param else max(float(want.double().pow(2).mean().sqrt()), 1e-30)
        rel = fp32_rel_err(got, want, floor)
        assert float(rel.max()) <= 1e-6, f"{what}: rel err {float(rel.max()):.3e}"


def compare_engines(got_eng, want_eng, what, exact: bool, body_only: int = 0):
    """Params and every state of two engines; ``exact`` demands bit equality.  ``body_only=w``
    leaves out the last ``numel % w`` elements of every tensor (the part a CPU kernel of vector
    width ``w`` handles in its scalar remainder loop)."""
    for i, (p, q) in enumerate(zip(got_eng.params, want_eng.params)):
        keep = p.numel() - (p.numel() % body_only if body_only else 0)
        if keep == 0:
            continue
        items = [("param", p, q)]
        for key in STATE_KEYS:
            a = got_eng.state[i].get(key) if got_eng.state[i] else None
            b = want_eng.state[i].get(key) if want_eng.state[i] else None
            assert (a is None) == (b is None), f"{what} tensor {i} {key}: present in one engine only"
            if a is not None:
                items.append((key, a, b))
        for key, a, b in items:
            label = f"{what} tensor {i} ({tuple(p.shape)}) {key}"
            a, b = a.detach().flatten()[:keep], b.detach().flatten()[:keep]
            if key == "kahan_comp":
                q = q.detach().flatten()[:keep]
            if exact:
                assert_bits_equal(a, b, label)
            else:
                assert_close_to_reference(a, b, label, param=q if key == "kahan_comp" else None,
                                          is_param=key in ("param", "la_param"))
