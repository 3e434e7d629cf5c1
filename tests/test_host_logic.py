"""Host-side behaviour of the Python layer that needs no GPU: constructor validation and
warnings (optimi/optimizer.py:15-72, adam.py:71-76), the state_dict layout, gradient-release
registration (optimi/gradientrelease.py:18-61), and the refusal to run anywhere but on the
HIP backend."""

import warnings

import pytest
import torch

import optimi_amd
from optimi_amd import functional as F
from optimi_amd.utils import debias, debias_beta

CLASSES = [optimi_amd.Adam, optimi_amd.AdamW, optimi_amd.Lion, optimi_amd.StableAdamW, optimi_amd.Adan,
           optimi_amd.SGD, optimi_amd.RAdam, optimi_amd.Ranger]
NO_BETAS = (optimi_amd.SGD,)
NO_EPS = (optimi_amd.Lion, optimi_amd.SGD)


def params():
    return [torch.nn.Parameter(torch.randn(4, 3)), torch.nn.Parameter(torch.randn(5))]


@pytest.mark.parametrize("cls", CLASSES)
def test_constructor_validation(cls):
    with pytest.raises(ValueError, match="learning rate"):
        cls(params(), lr=-1.0)
    with pytest.raises(ValueError, match="weight decay"):
        cls(params(), lr=1e-3, weight_decay=-0.1)
    if cls not in NO_BETAS:
        with pytest.raises(ValueError, match="beta1"):
            cls(params(), lr=1e-3, betas=(1.0, 0.9, 0.9)[: 3 if cls is optimi_amd.Adan else 2])
    else:
        with pytest.raises(ValueError, match="momentum"):
            cls(params(), lr=1e-3, momentum=1.0)
    with pytest.raises(ValueError, match="max_lr|maximum learning rate"):
        cls(params(), lr=1e-3, max_lr=-1.0)
    if cls not in NO_EPS:
        with pytest.raises(ValueError, match="epsilon"):
            cls(params(), lr=1e-3, eps=-1e-8)
    with pytest.warns(DeprecationWarning, match="foreach"):  # deprecated as in the reference; served by the HIP kernels
        cls(params(), lr=1e-3, foreach=True)
    with pytest.raises(ValueError, match="HIP backend"):
        cls(params(), lr=1e-3, triton=False)


@pytest.mark.parametrize("cls", CLASSES)
def test_group_keys_and_decouple_lr_defaults(cls):
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        opt = cls(params(), lr=3e-4, weight_decay=1e-2, decouple_lr=True)
    assert any("potentially high for decouple_lr=True" in str(w.message) for w in caught)
    g = opt.param_groups[0]
    assert g["max_lr"] == 3e-4 and g["decouple_lr"] is True and g["setup"] is False
    common = {"lr", "weight_decay", "decouple_lr", "max_lr", "kahan_sum", "foreach", "triton",
              "gradient_release", "setup", "params"}
    betas = {"beta1", "beta2"}
    extra = {optimi_amd.Adam: betas | {"eps", "decouple_wd"}, optimi_amd.AdamW: betas | {"eps", "decouple_wd"},
             optimi_amd.Lion: betas, optimi_amd.StableAdamW: betas | {"eps"},
             optimi_amd.Adan: betas | {"eps", "beta3", "adam_wd"},
             optimi_amd.SGD: {"momentum", "dampening", "decouple_wd", "torch_init"},
             optimi_amd.RAdam: betas | {"eps", "decouple_wd"},
             optimi_amd.Ranger: betas | {"eps", "decouple_wd", "k", "alpha"}}[cls]
    assert {k for k in g if not k.startswith("_")} - {"params"} >= (common | extra) - {"params"}
    assert set(opt.state_dict()["param_groups"][0]) >= (common | extra)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        cls(params(), lr=3e-4, weight_decay=1e-5, decouple_lr=True)  # low decay: no warning


def test_adamw_is_adam_with_decoupled_decay():
    opt = optimi_amd.AdamW(params(), lr=1e-3)
    assert isinstance(opt, optimi_amd.Adam) and opt.param_groups[0]["decouple_wd"] is True
    assert opt.param_groups[0]["weight_decay"] == 1e-2
    assert optimi_amd.Adam(params(), lr=1e-3).param_groups[0]["weight_decay"] == 0
    assert optimi_amd.Adan(params(), lr=1e-3).param_groups[0]["kahan_sum"] is False
    assert optimi_amd.Lion(params(), lr=1e-3).param_groups[0]["kahan_sum"] is None


@pytest.mark.parametrize("cls", CLASSES)
def test_cpu_parameters_are_refused_loudly(cls):
    ps = params()
    opt = cls(ps, lr=1e-3)
    for p in ps:
        p.grad = torch.randn_like(p)
    with pytest.raises(RuntimeError, match="HIP"):
        opt.step()
    ps = params()
    opt = cls(ps, lr=1e-3, triton=True)
    for p in ps:
        p.grad = torch.randn_like(p)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        opt.step()


def test_functional_forms_refuse_other_backends():
    p, g, m, v = (torch.zeros(4) for _ in range(4))
    step = torch.tensor(0, dtype=torch.int32)
    kw = dict(lr=1e-3, beta1=0.9, beta2=0.99, weight_decay=0.0, eps=1e-6, step=step)
    with pytest.raises(ValueError, match="only the fused HIP backend"):
        F.adamw([p], [g], [m], [v], **kw)
    with pytest.raises(RuntimeError, match="HIP devices only"):  # foreach=True selects the HIP kernels too
        F.adamw([p], [g], [m], [v], foreach=True, **kw)
    with pytest.raises(ValueError, match="cannot be used together"):
        F.adamw(p, g, m, v, foreach=True, gradient_release=True, **kw)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        F.adamw([p], [g], [m], [v], triton=True, **kw)
    assert int(step) == 0  # every rejected call left the counter where it was


def test_rejected_calls_do_not_advance_the_step_counter():
    """Tensors are validated before the counter moves, in every functional form that has one."""
    p, g, m, v, x, y = (torch.zeros(4) for _ in range(6))
    base = dict(lr=1e-3, beta1=0.9, beta2=0.99, weight_decay=0.0, eps=1e-6, triton=True)
    calls = {
        "adam": lambda s: F.adam([p], [g], [m], [v], decouple_wd=True, step=s, **base),
        "stableadamw": lambda s: F.stableadamw([p], [g], [m], [v], [x], step=s, **base),
        "adan": lambda s: F.adan([p], [g], [m], [v], [x], [y], beta3=0.99, step=s, **base),
        "radam": lambda s: F.radam([p], [g], [m], [v], decouple_wd=True, step=s, **base),
        "ranger": lambda s: F.ranger([p], [g], [m], [v], [x], k=6, alpha=0.5, decouple_wd=True, step=s, **base),
    }
    for name, call in calls.items():
        step = torch.tensor(3, dtype=torch.int32)
        with pytest.raises(RuntimeError, match="HIP devices only"):
            call(step)
        assert int(step) == 3, name
    # a gradient of another dtype and lists of unequal length are rejected before the counter moves, too
    step = torch.tensor(3, dtype=torch.int32)
    with pytest.raises(ValueError, match="got 1 parameters but a list of 2"):
        F.adam([p], [g, g], [m], [v], decouple_wd=True, step=step, **base)
    assert int(step) == 3


def test_step_without_gradients_is_a_noop_that_still_counts():
    ps = params()
    opt = optimi_amd.AdamW(ps, lr=1e-3)
    opt.step()
    assert int(opt.param_groups[0]["step"]) == 1 and len(opt.state) == 0
    sgd = optimi_amd.SGD(params(), lr=1e-3)
    sgd.step()
    assert "step" not in sgd.param_groups[0]


def test_gradient_release_setup_and_hooks():
    model = torch.nn.Sequential(torch.nn.Linear(4, 4), torch.nn.Linear(4, 2))
    model[0].bias.requires_grad_(False)
    plain = optimi_amd.AdamW(model.parameters(), lr=1e-3)
    with pytest.raises(ValueError, match="gradient_release=True"):
        optimi_amd.prepare_for_gradient_release(model, plain)
    with pytest.raises(TypeError, match="OptimiOptimizer"):
        optimi_amd.prepare_for_gradient_release(model, torch.optim.SGD(model.parameters(), lr=0.1))
    opt = optimi_amd.AdamW(model.parameters(), lr=1e-3, gradient_release=True)
    for group in opt.param_groups:
        assert group["foreach"] is False
        for p in group["params"]:
            assert opt.state[p]["group"] is group
    optimi_amd.prepare_for_gradient_release(model, opt)
    assert len(model._gradient_release_hooks) == 3  # the frozen bias gets none
    with pytest.raises(ValueError, match="already has post_accumulate_grad_hooks"):
        optimi_amd.prepare_for_gradient_release(model, opt)
    assert len(model._gradient_release_hooks) == 3
    optimi_amd.prepare_for_gradient_release(model, opt, ignore_existing_hooks=True)
    optimi_amd.remove_gradient_release(model)
    assert not hasattr(model, "_gradient_release_hooks")
    with pytest.warns(UserWarning, match="does not have any gradient release"):
        optimi_amd.remove_gradient_release(model)
    assert opt.optimizer_accumulation is False
    opt.optimizer_accumulation = True
    assert opt.optimizer_accumulation is True


def test_zero_grad_on_one_parameter():
    ps = params()
    opt = optimi_amd.AdamW(ps, lr=1e-3, gradient_release=True)
    for p in ps:
        p.grad = torch.ones_like(p)
    opt.zero_grad(param=ps[0])
    assert ps[0].grad is None and ps[1].grad is not None
    opt.zero_grad(set_to_none=False, param=ps[1])
    assert ps[1].grad is not None and not ps[1].grad.requires_grad
    opt.zero_grad()
    assert ps[1].grad is None


def test_scalar_helpers():
    assert debias(0.9, 1) == pytest.approx(0.1)
    assert debias_beta(0.9, 1) == 0.0
    assert debias_beta(0.9, 2) == pytest.approx(0.9 * (1 - 0.9) / (1 - 0.81))
