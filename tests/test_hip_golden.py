"""HIP kernels against the golden vectors the reference wrote (tests/golden/*.npz).

Each fixture is replayed twice through the C ABI – once with the whole-list entry points,
once with the per-tensor entry points – and every snapshot (params and all states after
steps 1, 3 and the last) is compared with what the reference's for-loop path produced.

Bar: bf16 tensors bit-exact, except StableAdamW, whose per-tensor mean is summed in a
different order than torch's (<= 1 bf16 ulp there; the Kahan buffer is judged in units of
the parameter's ulp).  fp32 tensors: |a-b| <= 1e-6 * max(|a|, |b|, floor); torch's CPU sqrt
is only faithfully rounded, so fp32 cannot be bit-exact.  Where the reference's own bf16 output
is not uniform (the scalar remainder loop of ATen's ``add_(x, alpha=...)``, used by SGD, RAdam,
Ranger and L2 decay) the last ``numel % 32`` elements are left out.  The floor covers elements that
cancel towards zero: 1e-2 for parameters (ten steps move a parameter by up to about 10 * lr, so
its rounding error is judged against that distance, i.e. |a-b| <= 1e-8 near zero) for StableAdamW's
parameters, a tenth of the tensor's RMS (about 2e-3) for every other optimizer's, and the tensor's RMS
for the moment states.  The worst error with no floor at all - |a-b| / max(|a|, |b|), and in fp32 ulps -
is collected per optimizer and printed at the end of the run (tests/conftest.py), so that a change in
it shows in the log even while the floored comparison still passes.
"""

import functools

import pytest
import torch

import golden_util as G

pytestmark = pytest.mark.gpu

FP32_REL = 1e-6
FP32_FLOOR_PARAM = 1e-2  # StableAdamW; every other optimizer is held to a tenth of the tensor's RMS (about 2e-3)


def compare_snapshot(name, key, got, want, param_want=None):
    keep = want.numel() - G.torch_tail(name, want.numel(), want.dtype)  # see golden_util.torch_tail
    got, want = got.flatten()[:keep], want.flatten()[:keep]
    if param_want is not None:
        param_want = param_want.flatten()[:keep]
    if want.dtype in (torch.bfloat16, torch.float16):
        ulp = G.bf16_ulp_diff(got, want)
        if "stableadamw" not in name:
            assert int(ulp.max()) == 0, f"{name} {key}: {int((ulp > 0).sum())} of {ulp.numel()} differ, max {int(ulp.max())} ulp"
        elif ".kahan_comp." in key:
            err = (got.float() - want.float()).abs() / G.bf16_ulp_of(param_want)
            assert float(err.max()) <= 1.0, f"{name} {key}: Kahan buffer off by {float(err.max())} param ulps"
        else:
            assert int(ulp.max()) <= 1, f"{name} {key}: max {int(ulp.max())} ulp"
    else:
        rms = max(float(want.double().pow(2).mean().sqrt()), 1e-30)
        is_param = ".param." in key or ".la_param." in key
        floor = (FP32_FLOOR_PARAM if "stableadamw" in name else 0.1 * rms) if is_param else rms
        rel = G.fp32_rel_err(got, want, floor)
        G.note_fp32_error(name, key, got, want)  # the unfloored figures, for the summary at the end of the run
        assert float(rel.max()) <= FP32_REL, f"{name} {key}: rel err {float(rel.max())}"


@pytest.mark.parametrize("multi", [True, False], ids=["multi", "single"])
@pytest.mark.parametrize("name", G.case_names())
def test_fixture(name, multi, hip_device):
    from hip_engine import HipRun

    fx = G.load(name)
    out = G.replay(name, fx, functools.partial(HipRun, multi=multi), device=hip_device)
    wanted = [k for k in fx if k.startswith("out.")]
    assert sorted(out) == sorted(wanted)
    for key in wanted:
        step, _, idx = key.split(".")[1], key.split(".")[2], key.split(".")[3]
        compare_snapshot(name, key, out[key], fx[key], fx.get(f"out.{step}.param.{idx}"))


@pytest.mark.parametrize("multi", [True, False], ids=["multi", "single"])
@pytest.mark.parametrize("name", G.case_names())
def test_fixture_through_a_driver_that_owes_the_oracle_nothing(name, multi, hip_device):
    """The same fixtures through ``PlainHipRun``: its state creation and scalar prologue share no
    code with ``oracle/`` (``HipRun`` inherits both from the oracle's driver)."""
    from hip_engine import PlainHipRun

    fx = G.load(name)
    out = G.replay(name, fx, functools.partial(PlainHipRun, multi=multi), device=hip_device)
    wanted = [k for k in fx if k.startswith("out.")]
    assert sorted(out) == sorted(wanted)
    for key in wanted:
        step, _, idx = key.split(".")[1], key.split(".")[2], key.split(".")[3]
        compare_snapshot(name, key, out[key], fx[key], fx.get(f"out.{step}.param.{idx}"))


class ClassRun:
    """The product path as a user drives it: the optimizer class with the fixture's constructor
    arguments, gradients put on ``.grad``, ``step()`` for whole-list cases and the registered
    native hook for gradient release."""

    def __init__(self, name, params, gradient_release=False, native=True, **kwargs):
        import optimi_amd

        cls = {"adam": optimi_amd.Adam, "adamw": optimi_amd.AdamW, "lion": optimi_amd.Lion,
               "stableadamw": optimi_amd.StableAdamW, "adan": optimi_amd.Adan, "sgd": optimi_amd.SGD,
               "radam": optimi_amd.RAdam, "ranger": optimi_amd.Ranger}[name]
        self.params = [torch.nn.Parameter(p) for p in params]
        self.opt = cls(self.params, gradient_release=gradient_release, **kwargs)
        self.opt.native_step = native
        self.hook = self.opt._native_hook() if (gradient_release and native) else None
        self.optimizer_accumulation = False

    @property
    def state(self):
        return [self.opt.state[p] if p in self.opt.state else None for p in self.params]

    def step(self, grads):
        for p, g in zip(self.params, grads):
            p.grad = g
        self.opt.step()
        self.opt.zero_grad()

    def step_param(self, i, grad):
        p = self.params[i]
        p.grad = grad
        self.opt.optimizer_accumulation = self.optimizer_accumulation
        if self.hook is not None:
            self.hook(p)
        else:
            self.opt.step(param=p)
            self.opt.zero_grad(param=p)
        assert p.grad is None


@pytest.mark.parametrize("native", [True, False], ids=["native_driver", "python_driver"])
@pytest.mark.parametrize("name", G.case_names(functional=False))
def test_fixture_through_the_optimizer_classes(name, native, hip_device):
    """Same constructor arguments and inputs as the reference was given, same bits out: the
    scalar prologue, lazy state creation and step counters of the product's Python and native
    drivers are held to the fixtures too, not only the kernels."""
    fx = G.load(name)
    out = G.replay(name, fx, functools.partial(ClassRun, native=native), device=hip_device)
    wanted = [k for k in fx if k.startswith("out.")]
    assert sorted(out) == sorted(wanted)
    for key in wanted:
        param_key = None
        if ".kahan_comp." in key:
            step, _, idx = key.split(".")[1:4]
            param_key = f"out.{step}.param.{idx}"
        compare_snapshot(name, key, out[key], fx[key], fx[param_key] if param_key else None)


@pytest.mark.parametrize("name", G.case_names())
def test_fixture_through_the_functional_forms(name, hip_device):
    """The eight public functional forms called directly, as the reference's functional API is
    called: lists for whole-list cases, bare tensors with ``gradient_release=True`` for release
    cases, no workspace passed in.  Same bar as the kernels."""
    from hip_engine import FunctionalRun

    fx = G.load(name)
    out = G.replay(name, fx, FunctionalRun, device=hip_device)
    wanted = [k for k in fx if k.startswith("out.")]
    assert sorted(out) == sorted(wanted)
    for key in wanted:
        step, _, idx = key.split(".")[1:4]
        compare_snapshot(name, key, out[key], fx[key], fx.get(f"out.{step}.param.{idx}"))
