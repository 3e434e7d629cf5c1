"""Optimizers with more than one parameter group (what ``param_groups_weight_decay`` produces):
every group keeps its own launch tables, so steps after the first upload nothing, and whether a
list is read with cached or with streaming loads is decided for the optimizer as a whole, not
per launch."""

import pytest
import torch

import golden_util as G
import optimi_amd
from optimi_amd import cabi
from oracle.forloop import ForLoopRun

pytestmark = pytest.mark.gpu


def two_groups(device, n_each=24, dtype=torch.bfloat16, seed=0):
    gen = torch.Generator().manual_seed(seed)
    mats = [torch.nn.Parameter((torch.randn(37 + i, 64, generator=gen) * 0.02).to(dtype).to(device)) for i in range(n_each)]
    vecs = [torch.nn.Parameter(torch.ones(64 + 8 * i, dtype=dtype, device=device)) for i in range(n_each)]
    return mats, vecs


@pytest.mark.parametrize("native", [True, False], ids=["native_walk", "python_walk"])
def test_each_group_keeps_its_tables_between_steps(hip_device, native):
    """Two groups of 24 tensors each (device tables, not the kernel-argument table): from the third
    step on - the first is set up in Python, the second fills the tables of whichever walk is in use -
    nothing is uploaded, one kernel per group, and the result is the for-loop oracle's bit for bit."""
    L = cabi.lib()
    mats, vecs = two_groups(hip_device)
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6)
    opt = optimi_amd.AdamW([{"params": mats, "weight_decay": 1e-2}, {"params": vecs, "weight_decay": 0.0}], **hyper)
    opt.native_step = native
    refs = [ForLoopRun("adamw", [p.detach().cpu().clone() for p in ps], weight_decay=wd, **hyper)
            for ps, wd in ((mats, 1e-2), (vecs, 0.0))]
    gen = torch.Generator().manual_seed(1)
    grads = [(torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype) for p in mats + vecs]
    dev_grads = [g.to(hip_device) for g in grads]  # the same buffers every step: the pointers in the tables do not move
    for it in range(6):
        for p, g in zip(mats + vecs, dev_grads):
            p.grad = g
        uploads, launches = L.optimi_hip_upload_count(), L.optimi_hip_launch_count()
        opt.step()
        if it >= 2:
            assert L.optimi_hip_upload_count() == uploads, f"step {it + 1} uploaded a table again"
        assert L.optimi_hip_launch_count() - launches == 2
        refs[0].step([g.clone() for g in grads[:len(mats)]])
        refs[1].step([g.clone() for g in grads[len(mats):]])
    torch.cuda.synchronize()
    for ref, ps in zip(refs, (mats, vecs)):
        for i, p in enumerate(ps):
            G.assert_bits_equal(p.detach().cpu(), ref.params[i], f"param {i}")
            for key in ("exp_avg", "exp_avg_sq", "kahan_comp"):
                G.assert_bits_equal(opt.state[p][key].cpu(), ref.state[i][key], f"{key} {i}")


@pytest.mark.parametrize("native", [True, False], ids=["native_walk", "python_walk"])
def test_gradients_that_alternate_between_two_sets_of_buffers_upload_nothing(hip_device, native):
    """``p.grad = fresh_tensor`` every step makes the allocator hand out two sets of blocks in turn
    (the new gradient exists before the old one is freed); so do double-buffered gradient buckets.
    A group keeps two tables on the device, so once both have been seen nothing is uploaded.  Three
    sets in rotation miss every time - results are the oracle's either way."""
    L = cabi.lib()
    mats, vecs = two_groups(hip_device, n_each=20)
    params = mats + vecs
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
    opt = optimi_amd.AdamW(params, **hyper)
    opt.native_step = native
    ref = ForLoopRun("adamw", [p.detach().cpu().clone() for p in params], **hyper)
    gen = torch.Generator().manual_seed(2)
    sets = [[(torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype) for p in params] for _ in range(3)]
    dev_sets = [[g.to(hip_device) for g in gs] for gs in sets]

    def step(k):
        for p, g in zip(params, dev_sets[k]):
            p.grad = g
        before = L.optimi_hip_upload_count()
        opt.step()
        ref.step([g.clone() for g in sets[k]])
        return L.optimi_hip_upload_count() - before

    for it in range(4):  # set-up steps: the Python walk's first step, then both tables of the walk in use
        step(it % 2)
    assert [step(it % 2) for it in range(6)] == [0] * 6, "alternating gradient buffers uploaded a table again"
    # three sets in rotation: the first of them is still on the device, after that one table (and no chunk map) per step
    assert [step(it % 3) for it in range(1, 7)] == [0, 1, 1, 1, 1, 1]
    torch.cuda.synchronize()
    for i, p in enumerate(params):
        G.assert_bits_equal(p.detach().cpu(), ref.params[i], f"param {i}")
        for key in ("exp_avg", "exp_avg_sq", "kahan_comp"):
            G.assert_bits_equal(opt.state[p][key].cpu(), ref.state[i][key], f"{key} {i}")


def test_load_state_dict_and_add_param_group_drop_the_cached_tables(hip_device):
    """The workspaces are keyed by the group dicts; a state_dict round trip replaces those, and the
    tables must follow (one more upload per group, none after)."""
    L = cabi.lib()
    mats, vecs = two_groups(hip_device, seed=3)
    opt = optimi_amd.AdamW([{"params": mats}, {"params": vecs, "weight_decay": 0.0}], lr=1e-3)
    grads = [torch.full_like(p, 1e-3) for p in mats + vecs]

    def step():
        for p, g in zip(mats + vecs, grads):
            p.grad = g
        before = L.optimi_hip_upload_count()
        opt.step()
        return L.optimi_hip_upload_count() - before

    step(), step()
    assert step() == 0
    opt.load_state_dict(opt.state_dict())
    assert step() > 0
    assert step() == 0
    extra = [torch.nn.Parameter(torch.zeros(100, dtype=torch.bfloat16, device=hip_device)) for _ in range(20)]
    opt.add_param_group({"params": extra})
    for p in extra:
        p.grad = torch.full_like(p, 1e-3)
    step(), step()
    assert step() == 0
    torch.cuda.synchronize()


def test_cached_loads_are_opt_in_and_decided_for_the_whole_optimizer(hip_device):
    """By default every list is streamed (a training loop sweeps the cache between steps).  With
    ``resident_lists = True`` a small model is read with cached loads - but the same small group beside a
    group that does not fit the cache is cold every time it is stepped, and stays streamed.  Both
    walks agree.  (Bits never depend on this: see test_resident_hint_changes_nothing.)"""
    L = cabi.lib()
    ext = optimi_amd.backend.ext()
    limit = ext.resident_bytes()
    assert limit == L.optimi_hip_resident_bytes() > 0

    def resident_launches(opt, params):
        for p in params:
            p.grad = torch.full_like(p, 1e-3)
        opt.step()  # the first step of a group is set up in Python; count a later one
        before = L.optimi_hip_resident_launch_count()
        opt.step()
        return L.optimi_hip_resident_launch_count() - before

    mats, vecs = two_groups(hip_device, seed=5)
    small = optimi_amd.AdamW([{"params": mats}, {"params": vecs, "weight_decay": 0.0}], lr=1e-3)
    assert not small._lists_are_resident()
    assert resident_launches(small, mats + vecs) == 0
    small.resident_lists = True
    assert small._lists_are_resident()
    assert resident_launches(small, mats + vecs) == 2
    small.native_step = False
    assert resident_launches(small, mats + vecs) == 2
    small.resident_lists = False
    assert resident_launches(small, mats + vecs) == 0

    # one bf16 tensor whose five arrays (parameter, gradient, two moments, Kahan buffer) exceed the limit
    big = torch.nn.Parameter(torch.zeros(limit // 10 + 4096, dtype=torch.bfloat16, device=hip_device))
    mats2, vecs2 = two_groups(hip_device, seed=6)
    large = optimi_amd.AdamW([{"params": [big] + mats2}, {"params": vecs2, "weight_decay": 0.0}], lr=1e-3)
    large.resident_lists = True
    assert not large._lists_are_resident()  # the hint is given, the optimizer as a whole does not fit
    assert resident_launches(large, [big] + mats2 + vecs2) == 0
    large.native_step = False
    assert resident_launches(large, [big] + mats2 + vecs2) == 0
    torch.cuda.synchronize()
