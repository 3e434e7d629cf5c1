"""Steps that must be refused are refused as Python exceptions, before anything moves: the step
counter, the parameters and the states are as they were, and the optimizer works again once the
cause is gone.  Whole-group steps through both walks, and the native gradient-release hook, whose
exception has to travel out of the autograd engine's backward pass."""

import pytest
import torch

import optimi_amd

pytestmark = pytest.mark.gpu


def model_and_opt(device, release=False, n=20, cls=None):
    gen = torch.Generator().manual_seed(5)
    model = torch.nn.Module()
    model.ps = torch.nn.ParameterList(
        [torch.nn.Parameter((torch.randn(50 + i, 8, generator=gen) * 0.02).bfloat16().to(device)) for i in range(n)])
    opt = (cls or optimi_amd.AdamW)(model.parameters(), lr=1e-3, gradient_release=release)
    if release:
        optimi_amd.prepare_for_gradient_release(model, opt)
    return model, opt


def snapshot(model, opt):
    out = []
    for p in model.ps:
        st = opt.state.get(p, {})
        out.append((p.detach().clone(), {k: (v.clone() if torch.is_tensor(v) else v) for k, v in st.items() if k != "group"}))
    return out


def assert_unchanged(model, opt, before):
    for p, (p0, st0) in zip(model.ps, before):
        assert torch.equal(p.detach(), p0)
        st = opt.state.get(p, {})
        for k, v in st0.items():
            if torch.is_tensor(v) and k in st and torch.is_tensor(st[k]) and st[k].shape == v.shape:
                assert torch.equal(st[k], v), k


@pytest.mark.parametrize("native", [True, False], ids=["native_walk", "python_walk"])
def test_a_state_of_the_wrong_size_refuses_the_whole_group_step(hip_device, native):
    model, opt = model_and_opt(hip_device)
    opt.native_step = native
    for _ in range(2):
        for p in model.ps:
            p.grad = torch.full_like(p, 1e-3)
        opt.step()
    torch.cuda.synchronize()
    victim = model.ps[7]
    good = opt.state[victim]["exp_avg"]
    opt.state[victim]["exp_avg"] = torch.zeros(5, dtype=torch.bfloat16, device=hip_device)
    before, count = snapshot(model, opt), int(opt.param_groups[0]["step"])
    for p in model.ps:
        p.grad = torch.full_like(p, 1e-3)
    with pytest.raises(RuntimeError, match="elements|size|strides"):
        opt.step()
    torch.cuda.synchronize()
    assert int(opt.param_groups[0]["step"]) == count, "a refused step moved the step counter"
    assert_unchanged(model, opt, before)
    opt.state[victim]["exp_avg"] = good
    opt.step()  # and it works again
    torch.cuda.synchronize()
    assert int(opt.param_groups[0]["step"]) == count + 1
    assert not torch.equal(model.ps[0].detach(), before[0][0])


def test_a_sparse_gradient_is_refused(hip_device):
    emb = torch.nn.Embedding(64, 16, sparse=True).to(hip_device)
    opt = optimi_amd.AdamW(emb.parameters(), lr=1e-3)
    emb(torch.tensor([1, 5], device=hip_device)).sum().backward()
    with pytest.raises(RuntimeError, match="sparse"):
        opt.step()
    # the second time the native walk is in charge (the group is set up by then only if a step succeeded; either way: refused)
    with pytest.raises(RuntimeError, match="sparse"):
        opt.step()


def test_an_error_in_the_native_hook_leaves_the_backward_pass_as_an_exception(hip_device):
    model, opt = model_and_opt(hip_device, release=True)
    x = torch.ones(8, device=hip_device, dtype=torch.bfloat16)

    def backward():
        sum((p @ x).sum() for p in model.ps).backward()

    backward()
    backward()
    torch.cuda.synchronize()
    victim = model.ps[3]
    good = opt.state[victim]["exp_avg_sq"]
    opt.state[victim]["exp_avg_sq"] = torch.zeros(3, dtype=torch.bfloat16, device=hip_device)
    steps_before = int(opt.state[victim]["step"])
    p_before = victim.detach().clone()
    with pytest.raises(RuntimeError, match="elements|size|strides"):
        backward()
    opt.zero_grad()  # launches what the other hooks had parked, drops what is left of the gradients
    torch.cuda.synchronize()
    assert int(opt.state[victim]["step"]) == steps_before, "the refused step moved the parameter's counter"
    assert torch.equal(victim.detach(), p_before)
    opt.state[victim]["exp_avg_sq"] = good
    backward()
    torch.cuda.synchronize()
    assert int(opt.state[victim]["step"]) == steps_before + 1
    assert not torch.equal(victim.detach(), p_before)
    assert all(p.grad is None for p in model.ps)
    optimi_amd.remove_gradient_release(model)


def test_the_hook_of_a_deleted_optimizer_says_so(hip_device):
    model, opt = model_and_opt(hip_device, release=True, n=3)
    hook = opt._native_hook()
    p = model.ps[0]
    p.grad = torch.full_like(p, 1e-3)
    hook(p)
    assert p.grad is None
    with pytest.raises(RuntimeError, match="takes the parameter"):
        hook(p, p)
    with pytest.raises(RuntimeError, match="takes the parameter"):
        hook(3)
    optimi_amd.remove_gradient_release(model)  # the model kept the optimizer alive
    del opt
    import gc
    gc.collect()
    p.grad = torch.full_like(p, 1e-3)
    with pytest.raises(RuntimeError, match="no longer exists"):
        hook(p)
    torch.cuda.synchronize()
