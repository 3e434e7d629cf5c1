"""The native step and the native gradient-release hook hold no references they do not give back:
after many steps the parameters, their gradients' owners, the group dict, the state dicts and the
state tensors have the reference counts they had after the first steps, and an optimizer that is
dropped is collected together with its native core."""

import gc
import sys
import weakref

import pytest
import torch

import optimi_amd

pytestmark = pytest.mark.gpu


def counts(model, opt):
    out = []
    for p in model.ps:
        st = opt.state[p]
        out.append((sys.getrefcount(p), sys.getrefcount(st), tuple(sys.getrefcount(v) for v in st.values())))
    out.append(tuple(sys.getrefcount(g) for g in opt.param_groups))
    out.append(sys.getrefcount(opt))
    return out


def build(device, release, cls, n=24):
    gen = torch.Generator().manual_seed(3)
    model = torch.nn.Module()
    model.ps = torch.nn.ParameterList(
        [torch.nn.Parameter((torch.randn(40 + i, 8, generator=gen) * 0.02).bfloat16().to(device)) for i in range(n)])
    opt = cls(model.parameters(), lr=1e-3, gradient_release=release)
    if release:
        optimi_amd.prepare_for_gradient_release(model, opt)
    return model, opt


@pytest.mark.parametrize("cls", [optimi_amd.AdamW, optimi_amd.StableAdamW, optimi_amd.Adan, optimi_amd.SGD], ids=lambda c: c.__name__)
@pytest.mark.parametrize("native", [True, False], ids=["native_walk", "python_walk"])
def test_whole_group_steps_keep_reference_counts(hip_device, cls, native):
    model, opt = build(hip_device, False, cls)
    opt.native_step = native

    def step():
        for p in model.ps:
            p.grad = torch.full_like(p, 1e-3)
        opt.step()
        opt.zero_grad()

    for _ in range(3):
        step()
    gc.collect()
    before = counts(model, opt)
    for _ in range(200):
        step()
    torch.cuda.synchronize()
    gc.collect()
    assert counts(model, opt) == before


@pytest.mark.parametrize("cls", [optimi_amd.AdamW, optimi_amd.StableAdamW, optimi_amd.Lion], ids=lambda c: c.__name__)
@pytest.mark.parametrize("coalesce", [True, False], ids=["queued", "per_tensor"])
def test_release_hooks_keep_reference_counts(hip_device, cls, coalesce):
    gen = torch.Generator().manual_seed(3)
    model = torch.nn.Module()
    model.ps = torch.nn.ParameterList(
        [torch.nn.Parameter((torch.randn(40 + i, 8, generator=gen) * 0.02).bfloat16().to(hip_device)) for i in range(24)])
    opt = cls(model.parameters(), lr=1e-3, gradient_release=True)
    if not coalesce:
        opt.gradient_release_coalesce = 0
    optimi_amd.prepare_for_gradient_release(model, opt)
    x = torch.ones(8, device=hip_device, dtype=torch.bfloat16)

    def backward(i):
        opt.optimizer_accumulation = (i % 4) != 3
        sum((p @ x).sum() for p in model.ps).backward()
        opt.step()
        opt.zero_grad()

    for i in range(4):
        backward(i)
    gc.collect()
    before = counts(model, opt)
    for i in range(200):
        backward(i)
    torch.cuda.synchronize()
    gc.collect()
    assert counts(model, opt) == before
    assert all(p.grad is None for p in model.ps)
    optimi_amd.remove_gradient_release(model)


def test_a_dropped_optimizer_is_collected_with_its_tensors(hip_device):
    model, opt = build(hip_device, True, optimi_amd.AdamW, n=6)
    x = torch.ones(8, device=hip_device, dtype=torch.bfloat16)
    sum((p @ x).sum() for p in model.ps).backward()
    opt.step()
    opt.zero_grad()
    for p in model.ps:
        p.grad = torch.full_like(p, 1e-3)
    torch.cuda.synchronize()
    state_tensor = weakref.ref(opt.state[model.ps[0]]["exp_avg"])
    opt_ref = weakref.ref(opt)
    optimi_amd.remove_gradient_release(model)
    del opt
    gc.collect()
    assert opt_ref() is None, "something keeps the optimizer alive after its hooks were removed"
    assert state_tensor() is None, "a state tensor outlived its optimizer"
