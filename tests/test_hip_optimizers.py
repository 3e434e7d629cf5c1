"""The optimizer classes on a HIP device against the CPU for-loop oracle, in the three
scenarios of the reference's own test runner (tests/runner.py:75-332): a normal training loop
with a state_dict round trip into a fresh optimizer, gradient release driven by real
post-accumulate-grad hooks (with redundant step()/zero_grad() calls thrown in), and
optimizer accumulation with ``(i + 1) % 4``.  A small MLP with a real backward pass supplies
the gradients; the oracle is fed the very same gradients, so the north-star tolerance applies
at every step, not only at the end.
"""

import io
import random

import pytest
import torch

import golden_util as G
import optimi_amd
from optimi_amd import cabi
from oracle.forloop import ForLoopRun

pytestmark = pytest.mark.gpu

CASES = {
    "adam": (optimi_amd.Adam, "adam", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)),
    "adamw": (optimi_amd.AdamW, "adamw", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)),
    "adamw_declr": (optimi_amd.AdamW, "adamw", dict(lr=1e-3, weight_decay=1e-5, decouple_lr=True)),
    "lion": (optimi_amd.Lion, "lion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)),
    "stableadamw": (optimi_amd.StableAdamW, "stableadamw", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)),
    "adan": (optimi_amd.Adan, "adan", dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2, kahan_sum=True)),
    "sgd": (optimi_amd.SGD, "sgd", dict(lr=1e-2, momentum=0.9, weight_decay=1e-2, decouple_wd=True)),
    "radam": (optimi_amd.RAdam, "radam", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, decouple_wd=True)),
    "ranger": (optimi_amd.Ranger, "ranger", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, k=3)),
}


class MLP(torch.nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        self.norm = torch.nn.LayerNorm(dim)
        self.fc1 = torch.nn.Linear(dim, hidden, bias=False)
        self.act = torch.nn.Mish()
        self.fc2 = torch.nn.Linear(hidden, 1, bias=False)

    def forward(self, x):
        return self.fc2(self.act(self.fc1(self.norm(x))))


def make(dtype, device, seed=0):
    torch.manual_seed(seed)
    model = MLP(128, 1000).to(dtype=dtype, device=device)
    return model, list(model.parameters())


def loss_step(model, dtype, device, gen):
    x = torch.randn(32, 128, generator=gen).to(dtype=dtype, device=device)
    y = torch.randn(32, 1, generator=gen).to(dtype=dtype, device=device)
    loss = torch.nn.functional.mse_loss(model(x), y)
    loss.backward()


def oracle_for(oname, params, hyper, **kw):
    hyper = dict(hyper)
    if oname == "adam":
        hyper.setdefault("decouple_wd", False)
    return ForLoopRun(oname, [p.detach().cpu().clone() for p in params], **hyper, **kw)


def compare(opt, params, ref, what):
    # bf16 SGD / RAdam / Ranger: the reference is not uniform over the last numel % 32 elements
    # (scalar remainder loop of ATen's add_(x, alpha=...)); those are left out
    cut = ref.name in ("sgd", "radam", "ranger") and params[0].dtype != torch.float32
    for i, p in enumerate(params):
        keep = p.numel() - (p.numel() % 32 if cut else 0)
        if keep == 0:
            continue
        body = lambda t: t.detach().flatten()[:keep]  # noqa: E731
        G.assert_close_to_reference(body(p), body(ref.params[i]), f"{what} param {i}", is_param=True)
        st = opt.state[p]
        for key in G.STATE_KEYS:
            want = ref.state[i].get(key) if ref.state[i] else None
            if want is None:
                continue
            G.assert_close_to_reference(body(st[key]), body(want), f"{what} {key} {i}",
                                        param=body(ref.params[i]) if key == "kahan_comp" else None,
                                        is_param=key == "la_param")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16], ids=["bf16", "fp32", "fp16"])
@pytest.mark.parametrize("case", list(CASES))
def test_normal_with_state_dict_roundtrip(case, dtype, hip_device):
    cls, oname, hyper = CASES[case]
    model, params = make(dtype, hip_device)
    opt = cls(params, **hyper)
    ref = oracle_for(oname, params, hyper)
    gen = torch.Generator().manual_seed(1)
    for it in range(12):
        loss_step(model, dtype, hip_device, gen)
        grads = [p.grad.detach().cpu().clone() for p in params]
        opt.step()
        opt.zero_grad()
        ref.step(grads)
        compare(opt, params, ref, f"{case} it {it}")
        if it in (3, 7):  # checkpoint into a fresh optimizer, as tests/runner.py:244-251 does
            blob = io.BytesIO()
            torch.save(opt.state_dict(), blob)
            blob.seek(0)
            fresh = cls(params, **hyper)
            fresh.load_state_dict(torch.load(blob, weights_only=True))
            opt = fresh
    sd = opt.state_dict()
    per_param = sd["state"][0]
    assert "exp_avg" in per_param and "kahan_comp" in per_param
    assert all(not k.startswith("_") for k in sd["param_groups"][0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
@pytest.mark.parametrize("accumulate", [False, True], ids=["release", "accumulation"])
@pytest.mark.parametrize("case", ["adamw", "lion", "stableadamw", "adan", "sgd", "radam", "ranger"])
def test_gradient_release(case, accumulate, dtype, hip_device):
    cls, oname, hyper = CASES[case]
    model, params = make(dtype, hip_device)
    opt = cls(params, gradient_release=True, **hyper)
    optimi_amd.prepare_for_gradient_release(model, opt)
    ref = oracle_for(oname, params, hyper, gradient_release=True)
    seen = {}
    for i, p in enumerate(params):
        p.register_hook(lambda g, i=i: seen.__setitem__(i, g.detach().cpu().clone()))
    gen = torch.Generator().manual_seed(2)
    rnd = random.Random(3)
    for it in range(12):
        acc = accumulate and (it + 1) % 4 != 0
        opt.optimizer_accumulation = ref.optimizer_accumulation = acc
        seen.clear()
        loss_step(model, dtype, hip_device, gen)
        assert all(p.grad is None for p in params), "gradient release must free the gradients"
        if rnd.random() < 0.5:  # a plain step()/zero_grad() after the hooks ran is a harmless no-op
            opt.step()
            opt.zero_grad()
        for i in range(len(params)):
            ref.step_param(i, seen[i])
        compare(opt, params, ref, f"{case} it {it}")
    optimi_amd.remove_gradient_release(model)
    if oname not in ("lion", "sgd"):
        assert all(int(opt.state[p]["step"]) == 12 for p in params)


def test_two_param_groups_and_mixed_dtypes(hip_device):
    """A bf16 model with fp32 norm weights, one of them in the decay group beside the bf16 matrices, the
    other in a no-decay group of its own: one launch per group, whatever the dtypes in it."""
    torch.manual_seed(0)
    w = [torch.nn.Parameter((torch.randn(300, 70) * 0.02).to(torch.bfloat16).to(hip_device)) for _ in range(3)]
    n = [torch.nn.Parameter(torch.ones(70, device=hip_device)) for _ in range(2)]
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6)
    opt = optimi_amd.AdamW([{"params": w + n[:1], "weight_decay": 1e-2}, {"params": n[1:], "weight_decay": 0.0}], **hyper)
    ref_decay = ForLoopRun("adamw", [p.detach().cpu().clone() for p in w + n[:1]], weight_decay=1e-2, **hyper)
    ref_plain = ForLoopRun("adamw", [p.detach().cpu().clone() for p in n[1:]], weight_decay=0.0, **hyper)
    gen = torch.Generator().manual_seed(5)
    for _ in range(5):
        for p in w + n:
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype).to(hip_device)
        ref_decay.step([p.grad.cpu().clone() for p in w + n[:1]])
        ref_plain.step([p.grad.cpu().clone() for p in n[1:]])
        before = cabi.lib().optimi_hip_launch_count()
        opt.step()
        assert cabi.lib().optimi_hip_launch_count() - before == 2, "one kernel launch per parameter group"
        opt.zero_grad()
    for p, q in zip(w + n[:1], ref_decay.params):
        G.assert_close_to_reference(p, q, "decay group", is_param=True)
    G.assert_close_to_reference(n[1], ref_plain.params[0], "no-decay group", is_param=True)
    assert opt.state[w[0]]["kahan_comp"].shape == w[0].shape
    # fp32 parameters carry no Kahan buffer: None when the backend was resolved lazily on the first
    # step (optimi/adam.py:103-106 runs before :138-139), a 1-element placeholder with triton=True
    k = opt.state[n[0]]["kahan_comp"]
    assert k is None or k.numel() == 1


def test_noncontiguous_gradient_is_relaid(hip_device):
    p = torch.nn.Parameter((torch.randn(64, 48) * 0.02).to(hip_device))
    ref = ForLoopRun("adamw", [p.detach().cpu().clone()], lr=1e-3, weight_decay=1e-2)
    opt = optimi_amd.AdamW([p], lr=1e-3)
    g = (torch.randn(48, 64) * 1e-3).to(hip_device).t()  # same shape as p, transposed strides
    assert g.stride() != p.stride()
    p.grad = g
    opt.step()
    ref.step([g.cpu().contiguous()])
    G.assert_close_to_reference(p, ref.params[0], "strided grad", is_param=True)


@pytest.mark.parametrize("case", ["adamw", "adamw_declr", "lion", "stableadamw", "adan", "sgd", "radam", "ranger"])
def test_release_fast_path_equals_public_step(case, hip_device):
    """The hook's one-call native path and ``step(param=p); zero_grad(param=p)`` give the same bits,
    including the accumulate-only micro-steps and the per-parameter step counters."""
    cls, _, hyper = CASES[case]
    torch.manual_seed(0)
    p0 = [(torch.randn(s) * 0.02).bfloat16().to(hip_device) for s in [(300, 70), (8200,), (5,)]]
    a = [torch.nn.Parameter(p.clone()) for p in p0]
    b = [torch.nn.Parameter(p.clone()) for p in p0]
    fast, public = cls(a, gradient_release=True, **hyper), cls(b, gradient_release=True, **hyper)
    gen = torch.Generator().manual_seed(9)
    for it in range(8):
        fast.optimizer_accumulation = public.optimizer_accumulation = (it + 1) % 4 != 0
        for pa, pb in zip(reversed(a), reversed(b)):
            g = (torch.randn(pa.shape, generator=gen) * 1e-3).bfloat16().to(hip_device)
            pa.grad, pb.grad = g.clone(), g.clone()
            fast._release(pa)
            public.step(param=pb)
            public.zero_grad(param=pb)
            assert pa.grad is None and pb.grad is None
    for pa, pb in zip(a, b):
        G.assert_bits_equal(pa, pb, f"{case} param")
        for key, val in fast.state[pa].items():
            if torch.is_tensor(val) and key != "group":
                G.assert_bits_equal(val, public.state[pb][key], f"{case} {key}") if val.is_cuda else None
        if "step" in fast.state[pa]:
            assert int(fast.state[pa]["step"]) == int(public.state[pb]["step"]) == 8
    assert list(fast.state[a[0]].keys()) == list(public.state[b[0]].keys())


def test_step_hooks_still_fire_under_gradient_release(hip_device):
    model, params = make(torch.bfloat16, hip_device)
    opt = optimi_amd.AdamW(params, lr=1e-3, gradient_release=True)
    optimi_amd.prepare_for_gradient_release(model, opt)
    calls = []
    handle = opt.register_step_post_hook(lambda o, args, kwargs: calls.append(kwargs.get("param")))
    loss_step(model, torch.bfloat16, hip_device, torch.Generator().manual_seed(0))
    assert len(calls) == len(params) and all(c is not None for c in calls)
    handle.remove()
    loss_step(model, torch.bfloat16, hip_device, torch.Generator().manual_seed(1))
    assert len(calls) == len(params)
    optimi_amd.remove_gradient_release(model)


class ManySmall(torch.nn.Module):
    """Parameters of many sizes, most below the coalescing limit, two above it, two of them fp32;
    the loss gives every parameter a dense, non-trivial gradient."""

    SIZES = [5, 64, 513, 4096, 70000, 8191, 1, 300, 65536, 65537, 1000, 17, 2048, 9, 129, 33000]

    def __init__(self, device, seed=0):
        super().__init__()
        gen = torch.Generator().manual_seed(seed)
        self.ps = torch.nn.ParameterList()
        for i, n in enumerate(self.SIZES):
            dt = torch.float32 if i in (3, 11) else torch.bfloat16
            self.ps.append(torch.nn.Parameter((torch.randn(n, generator=gen) * 0.02).to(dt).to(device)))
        self.ws = [(torch.randn(n, generator=gen) * 1e-3).to(device) for n in self.SIZES]

    def forward(self, scale):
        return sum((p.float() * w).sum() for p, w in zip(self.ps, self.ws)) * scale


@pytest.mark.parametrize("max_tensors", [1024, 3], ids=["one_flush", "flush_every_3"])
@pytest.mark.parametrize("case", ["adamw", "adamw_declr", "lion", "stableadamw", "adan", "sgd", "radam", "ranger"])
def test_coalesced_release_equals_per_tensor_launches(case, max_tensors, hip_device):
    """Gradient release with small tensors parked and launched as lists (the default) gives the
    bits of one launch per tensor from each hook, across accumulate-only and full steps, two
    dtypes and tensors on both sides of the size limit."""
    cls, _, hyper = CASES[case]
    a, b = ManySmall(hip_device), ManySmall(hip_device)
    parked, direct = cls(a.parameters(), gradient_release=True, **hyper), cls(b.parameters(), gradient_release=True, **hyper)
    parked._QUEUE_MAX_TENSORS = max_tensors
    parked.gradient_release_coalesce = 65536  # ManySmall has tensors on both sides of this limit
    direct.gradient_release_coalesce = 0
    optimi_amd.prepare_for_gradient_release(a, parked)
    optimi_amd.prepare_for_gradient_release(b, direct)
    for it in range(8):
        parked.optimizer_accumulation = direct.optimizer_accumulation = (it + 1) % 4 != 0
        for model in (a, b):
            model(1.0 + it).backward()
        assert parked._release_queue.pending() == 0 and direct._release_queue is None
        assert all(p.grad is None for p in a.parameters())
    for i, (pa, pb) in enumerate(zip(a.parameters(), b.parameters())):
        G.assert_bits_equal(pa, pb, f"{case} param {i}")
        assert list(parked.state[pa].keys()) == list(direct.state[pb].keys())
        for key, val in parked.state[pa].items():
            if torch.is_tensor(val) and val.is_cuda and val.is_floating_point():
                G.assert_bits_equal(val, direct.state[pb][key], f"{case} {key} {i}")
        if "step" in parked.state[pa]:
            assert int(parked.state[pa]["step"]) == int(direct.state[pb]["step"]) == 8
    assert not torch.equal(next(a.parameters()), ManySmall(hip_device).ps[0]), "nothing was stepped"
    optimi_amd.remove_gradient_release(a)
    optimi_amd.remove_gradient_release(b)


def test_release_flush_is_ordered_before_the_callers_next_work(hip_device):
    """Forward on a side stream, backward() called on the default stream: the autograd engine
    runs the hooks on the side stream (where the parameters were used) and makes the default
    stream wait for it before the final callbacks run.  The flush of the parked steps happens in
    such a callback; work the caller enqueues on the default stream right after backward() - here
    a copy of every parameter - must see its result.  The side stream is kept busy so that a
    flush left on it would still be waiting when the copies run."""
    a, b = ManySmall(hip_device), ManySmall(hip_device)
    hyper = CASES["adamw"][2]
    parked = optimi_amd.AdamW(a.parameters(), gradient_release=True, **hyper)
    direct = optimi_amd.AdamW(b.parameters(), gradient_release=True, **hyper)
    direct.gradient_release_coalesce = 0
    optimi_amd.prepare_for_gradient_release(a, parked)
    optimi_amd.prepare_for_gradient_release(b, direct)
    side = torch.cuda.Stream()
    ballast = torch.randn(4096, 4096, device=hip_device)
    torch.cuda.synchronize()
    for it in range(6):
        snaps = []
        for model in (a, b):
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                loss = model(1.0 + it)
                for _ in range(8):
                    ballast @ ballast  # keeps the side stream busy past the end of backward()
            loss.backward()
            snaps.append([p.detach().clone() for p in model.parameters()])  # default stream, no sync in between
        assert parked._release_queue.pending() == 0
        torch.cuda.synchronize()
        for i, (x, y) in enumerate(zip(*snaps)):
            G.assert_bits_equal(x, y, f"pass {it} param {i} as the default stream saw it right after backward()")
    assert not torch.equal(next(a.parameters()), ManySmall(hip_device).ps[0]), "nothing was stepped"
    optimi_amd.remove_gradient_release(a)
    optimi_amd.remove_gradient_release(b)


def test_release_outside_a_backward_pass_launches_at_once(hip_device):
    """Steps are parked only inside a backward pass (its end launches them); a hook body called
    by hand launches its tensor directly."""
    p = torch.nn.Parameter((torch.randn(1000) * 0.02).bfloat16().to(hip_device))
    before = p.detach().clone()
    opt = optimi_amd.AdamW([p], lr=1e-3, gradient_release=True)
    p.grad = torch.full_like(p, 1e-3)
    opt._release(p)
    assert opt._release_queue.pending() == 0 and p.grad is None
    assert not torch.equal(p.detach(), before)
    assert int(opt.state_dict()["state"][0]["step"]) == 1


@pytest.mark.parametrize("case", ["adamw", "lion", "stableadamw", "adan", "sgd", "radam", "ranger"])
def test_native_hook_equals_python_hook(case, hip_device):
    """The registered (native) hook against the Python hook body on the same gradients, with a
    learning-rate change, a state_dict round trip into the live optimizer and a replaced state
    tensor in between: the native hook re-reads hyper-parameters every call and notices both."""
    from functools import partial

    from optimi_amd.gradient_release import _gradient_release_hook

    cls, _, hyper = CASES[case]
    a, b = ManySmall(hip_device), ManySmall(hip_device)
    native, python = cls(a.parameters(), gradient_release=True, **hyper), cls(b.parameters(), gradient_release=True, **hyper)
    optimi_amd.prepare_for_gradient_release(a, native)
    handles = [p.register_post_accumulate_grad_hook(partial(_gradient_release_hook, optimizer=python)) for p in b.parameters()]
    for it in range(9):
        native.optimizer_accumulation = python.optimizer_accumulation = it in (1, 2)
        if it == 3:
            for opt in (native, python):
                opt.param_groups[0]["lr"] *= 0.5
        if it == 5:
            for opt in (native, python):
                opt.load_state_dict(opt.state_dict())
        if it == 7:  # a state tensor replaced behind the optimizer's back
            for opt, model in ((native, a), (python, b)):
                st = opt.state[model.ps[4]]
                st["exp_avg"] = st["exp_avg"].clone().mul_(0.5)
        for model in (a, b):
            model(1.0 + it).backward()
        assert all(p.grad is None for p in a.parameters()) and all(p.grad is None for p in b.parameters())
    for i, (pa, pb) in enumerate(zip(a.parameters(), b.parameters())):
        G.assert_bits_equal(pa, pb, f"{case} param {i}")
        assert list(native.state[pa].keys()) == list(python.state[pb].keys())
        for key, val in native.state[pa].items():
            if torch.is_tensor(val) and val.is_cuda and val.is_floating_point():
                G.assert_bits_equal(val, python.state[pb][key], f"{case} {key} {i}")
        if "step" in native.state[pa]:
            assert int(native.state[pa]["step"]) == int(python.state[pb]["step"]) == 9
    optimi_amd.remove_gradient_release(a)
    for h in handles:
        h.remove()


def test_hooks_do_not_keep_model_or_optimizer_alive(hip_device):
    import gc
    import weakref

    model = ManySmall(hip_device)
    opt = optimi_amd.AdamW(model.parameters(), lr=1e-3, gradient_release=True)
    optimi_amd.prepare_for_gradient_release(model, opt)
    model(1.0).backward()
    refs = [weakref.ref(model), weakref.ref(opt), weakref.ref(model.ps[0])]
    del model, opt
    gc.collect()
    assert all(r() is None for r in refs)


@pytest.mark.parametrize("case", list(CASES))
def test_native_group_step_equals_python_walk(case, hip_device):
    """step() with the parameter walk in native code against the Python walk (native_step=False):
    two groups, two dtypes, parameters whose gradient is missing on some steps or arrives late,
    a learning-rate change, a state_dict round trip into the live optimizer, a replaced state
    tensor, and a step on which nothing has a gradient (the step counter still advances)."""
    cls, _, hyper = CASES[case]
    a, b = ManySmall(hip_device), ManySmall(hip_device)

    def build(model):
        ps = list(model.parameters())
        return cls([{"params": ps[:9]}, {"params": ps[9:], "weight_decay": 0.0}], **hyper)

    native, python = build(a), build(b)
    python.native_step = False
    gen = torch.Generator().manual_seed(4)
    for it in range(10):
        grads = [(torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype).to(hip_device) for p in a.parameters()]
        if it == 3:
            for opt in (native, python):
                opt.param_groups[0]["lr"] *= 0.5
        if it == 5:
            for opt in (native, python):
                opt.load_state_dict(opt.state_dict())
        if it == 7:
            for opt, model in ((native, a), (python, b)):
                st = opt.state[model.ps[4]]
                st["exp_avg"] = st["exp_avg"].clone().mul_(0.5)
        for model in (a, b):
            for i, (p, g) in enumerate(zip(model.parameters(), grads)):
                late = i == 2 and it < 4            # first gradient on the fifth step
                skipped = i == 6 and it % 3 == 1    # no gradient now and then
                p.grad = None if (late or skipped or it == 8) else g.clone()
        native.step()
        python.step()
    for i, (pa, pb) in enumerate(zip(a.parameters(), b.parameters())):
        G.assert_bits_equal(pa, pb, f"{case} param {i}")
        assert list(native.state[pa].keys()) == list(python.state[pb].keys())
        for key, val in native.state[pa].items():
            if torch.is_tensor(val) and val.is_cuda and val.is_floating_point():
                G.assert_bits_equal(val, python.state[pb][key], f"{case} {key} {i}")
    for ga, gb in zip(native.param_groups, python.param_groups):
        if "step" in ga:
            assert int(ga["step"]) == int(gb["step"]) == 10
    assert not torch.equal(a.ps[0], ManySmall(hip_device).ps[0]), "nothing was stepped"


def test_step_hooks_and_profiler_ranges_survive_the_fast_step(hip_device):
    """step() skips torch's wrapper only when it has nothing to do: hooks registered later fire,
    with the arguments torch's wrapper would hand them, and a profiler sees the step's range."""
    model, params = make(torch.bfloat16, hip_device)
    opt = optimi_amd.AdamW(params, lr=1e-3)
    loss_step(model, torch.bfloat16, hip_device, torch.Generator().manual_seed(0))
    opt.step()
    seen = []
    pre = opt.register_step_pre_hook(lambda o, args, kwargs: seen.append(("pre", o is opt)))
    post = opt.register_step_post_hook(lambda o, args, kwargs: seen.append(("post", kwargs.get("param"))))
    opt.step()
    assert seen == [("pre", True), ("post", None)]
    pre.remove()
    post.remove()
    opt.step()
    assert len(seen) == 2
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU]) as prof:
        opt.step()
    assert any("Optimizer.step#AdamW.step" in e.name for e in prof.events())
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("error")  # the scheduler warns about step order if its wrapper did not see the step
        sched = torch.optim.lr_scheduler.LambdaLR(opt, lambda e: 0.5)
        opt.step()
        sched.step()
    assert opt.param_groups[0]["lr"] == 5e-4


def test_foreach_true_selects_the_hip_kernels(hip_device):
    """The reference's other accelerated selector: deprecated, accepted, same kernels and results
    as triton=True; with gradient release it is switched off with a warning, as in the reference."""
    import warnings

    a, b = ManySmall(hip_device), ManySmall(hip_device)
    with pytest.warns(DeprecationWarning, match="foreach"):
        via_foreach = optimi_amd.AdamW(a.parameters(), lr=1e-3, foreach=True)
    via_triton = optimi_amd.AdamW(b.parameters(), lr=1e-3, triton=True)
    for it in range(3):
        for model, opt in ((a, via_foreach), (b, via_triton)):
            model(1.0 + it).backward()
            opt.step()
            opt.zero_grad()
    for pa, pb in zip(a.parameters(), b.parameters()):
        G.assert_bits_equal(pa, pb, "foreach=True vs triton=True")
    assert via_foreach.param_groups[0]["foreach"] is True
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        opt = optimi_amd.AdamW(a.parameters(), lr=1e-3, foreach=True, gradient_release=True)
    assert opt.param_groups[0]["foreach"] is False


def test_add_param_group_after_steps(hip_device):
    """A group added later (layers unfrozen during fine-tuning) starts its own step counter at zero
    (optimi/adam.py:134-136: the counter is created at the group's first step) and takes the
    constructor's defaults for what it does not set."""
    torch.manual_seed(3)
    a = [torch.nn.Parameter((torch.randn(130, 40) * 0.02).to(torch.bfloat16).to(hip_device)) for _ in range(2)]
    b = [torch.nn.Parameter((torch.randn(77) * 0.02).to(hip_device))]
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6)
    opt = optimi_amd.AdamW(a, weight_decay=1e-2, **hyper)
    ref_a = ForLoopRun("adamw", [p.detach().cpu().clone() for p in a], weight_decay=1e-2, **hyper)
    ref_b = ForLoopRun("adamw", [p.detach().cpu().clone() for p in b], weight_decay=0.0, **hyper)
    gen = torch.Generator().manual_seed(4)

    def grads_for(ps):
        for p in ps:
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype).to(hip_device)
        return [p.grad.cpu().clone() for p in ps]

    for _ in range(3):
        ref_a.step(grads_for(a))
        opt.step()
        opt.zero_grad()
    opt.add_param_group({"params": b, "weight_decay": 0.0})
    for _ in range(4):
        ga, gb = grads_for(a), grads_for(b)
        ref_a.step(ga)
        ref_b.step(gb)
        opt.step()
        opt.zero_grad()
    assert int(opt.param_groups[0]["step"]) == 7 and int(opt.param_groups[1]["step"]) == 4
    for p, q in zip(a, ref_a.params):
        G.assert_close_to_reference(p, q, "first group", is_param=True)
    G.assert_close_to_reference(b[0], ref_b.params[0], "group added later", is_param=True)


@pytest.mark.parametrize("case", list(CASES))
def test_mixed_group_with_state_dict_roundtrip(case, hip_device):
    """One parameter group of bf16 matrices and fp32 vectors (what ``to_low_precision`` leaves
    behind), checkpointed into a fresh optimizer twice on the way: states of both dtypes, the
    1-element Kahan placeholders of the fp32 tensors and the group's step counter survive, and
    every tensor keeps following the reference's for-loop path."""
    cls, oname, hyper = CASES[case]
    gen = torch.Generator().manual_seed(9)
    shapes = [(96, 64), (64,), (200, 32), (32,)]
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(torch.bfloat16 if len(s) == 2 else torch.float32)
                                 .to(hip_device)) for s in shapes]
    opt = cls(params, **hyper)
    ref = oracle_for(oname, params, hyper)
    for it in range(10):
        for p in params:
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype).to(hip_device)
        grads = [p.grad.detach().cpu().clone() for p in params]
        opt.step()
        opt.zero_grad()
        ref.step(grads)
        compare(opt, params, ref, f"{case} mixed it {it}")
        if it in (2, 6):
            blob = io.BytesIO()
            torch.save(opt.state_dict(), blob)
            blob.seek(0)
            fresh = cls(params, **hyper)
            fresh.load_state_dict(torch.load(blob, weights_only=True))
            opt = fresh
    assert opt.state[params[0]]["exp_avg"].dtype == torch.bfloat16 and opt.state[params[1]]["exp_avg"].dtype == torch.float32


@pytest.mark.parametrize("release", [False, True], ids=["step", "gradient_release"])
def test_zero_dim_and_empty_parameters(release, hip_device):
    """A 0-dim parameter (a learnable temperature) and a parameter without elements beside ordinary
    ones: both calling forms accept them, the former is stepped, the latter is left alone."""
    gen = torch.Generator().manual_seed(12)
    shapes = [(), (0, 7), (50, 3), (0,)]
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.5).to(hip_device)) for s in shapes]
    hyper = dict(lr=1e-2, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
    opt = optimi_amd.AdamW(params, gradient_release=release, **hyper)
    ref = ForLoopRun("adamw", [p.detach().cpu().clone() for p in params], gradient_release=release, **hyper)
    hook = opt._native_hook() if release else None
    for _ in range(4):
        grads = [(torch.randn(s, generator=gen) * 1e-2) for s in shapes]
        if release:
            for i in reversed(range(len(params))):
                params[i].grad = grads[i].to(hip_device)
                hook(params[i])
                ref.step_param(i, grads[i].clone())
        else:
            for p, g in zip(params, grads):
                p.grad = g.to(hip_device)
            opt.step()
            opt.zero_grad()
            ref.step([g.clone() for g in grads])
    opt.step()  # under gradient release: launches whatever is still parked
    torch.cuda.synchronize()
    for i, (p, q) in enumerate(zip(params, ref.params)):
        assert p.shape == q.shape
        if p.numel():
            G.assert_close_to_reference(p, q, f"param {i} of shape {tuple(p.shape)}", is_param=True)
    # a group that holds nothing but empty low-precision parameters (Kahan buffers without an address)
    hollow = [torch.nn.Parameter(torch.zeros(s, dtype=torch.bfloat16, device=hip_device)) for s in [(0, 4), (0,)]]
    opt = optimi_amd.AdamW(hollow, gradient_release=release, **hyper)
    hook = opt._native_hook() if release else None
    for _ in range(3):
        for p in hollow:
            p.grad = torch.zeros_like(p)
            if release:
                hook(p)
        opt.step()
        opt.zero_grad()
    torch.cuda.synchronize()


@pytest.mark.parametrize("n_params", [6, 24], ids=["kernel_argument_table", "device_tables"])
@pytest.mark.parametrize("case", ["adamw", "stableadamw", "adan"])
def test_changing_subset_of_gradients_and_a_moving_learning_rate(case, n_params, hip_device):
    """Steps on which only some parameters have a gradient (frozen branches, unused heads) and a
    learning rate a scheduler moves every step: the launch list changes from step to step, the
    group's one step counter still advances for everyone (optimi/adam.py:164-182), and parameters
    without a gradient keep their values and states."""
    cls, oname, hyper = CASES[case]
    gen = torch.Generator().manual_seed(21)
    shapes = [[(40, 30), (8200,), (64,), (3, 5, 7)][i % 4] for i in range(n_params)]
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(torch.bfloat16).to(hip_device)) for s in shapes]
    opt = cls(params, **hyper)
    ref = oracle_for(oname, params, hyper)
    sched = torch.optim.lr_scheduler.LambdaLR(opt, lambda step: 1.0 / (1.0 + 0.25 * step))
    base_lr = hyper["lr"]
    for it in range(8):
        present = [(i + it) % 3 != 0 for i in range(n_params)]  # two thirds of the parameters; a third is first seen on the second step
        grads = []
        for p, on in zip(params, present):
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype).to(hip_device) if on else None
            grads.append(p.grad.detach().cpu().clone() if on else None)
        ref.hyper["lr"] = base_lr / (1.0 + 0.25 * it)
        if ref.hyper.get("decouple_lr"):
            ref.hyper["max_lr"] = base_lr
        opt.step()
        sched.step()
        opt.zero_grad()
        ref.step(grads)
    compare(opt, params, ref, f"{case} changing subsets")


@pytest.mark.parametrize("case", ["adamw", "stableadamw", "ranger"])
def test_deepcopy_continues_like_the_original(case, hip_device):
    """``copy.deepcopy`` of an optimizer (what EMA and checkpointing helpers do) copies parameters
    and states and must leave the launch workspaces behind: original and copy then step their own
    parameters to the same bits."""
    import copy

    cls, _, hyper = CASES[case]
    gen = torch.Generator().manual_seed(31)
    shapes = [(40, 30), (8200,), (64,)] * 7  # 21 tensors: device tables
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(torch.bfloat16).to(hip_device)) for s in shapes]
    opt = cls(params, **hyper)

    def run(optimizer, grads):
        for p, g in zip(optimizer.param_groups[0]["params"], grads):
            p.grad = g.clone()
        optimizer.step()
        optimizer.zero_grad()

    def draw():
        return [(torch.randn(s, generator=gen) * 1e-3).to(torch.bfloat16).to(hip_device) for s in shapes]

    for _ in range(3):
        run(opt, draw())
    twin = copy.deepcopy(opt)
    twin_params = twin.param_groups[0]["params"]
    assert all(a is not b and a.data_ptr() != b.data_ptr() for a, b in zip(params, twin_params))
    for _ in range(4):
        grads = draw()
        run(opt, grads)
        run(twin, grads)
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(params, twin_params)):
        G.assert_bits_equal(a, b, f"{case} param {i}")
        for key in G.STATE_KEYS:
            if key in opt.state[a] and torch.is_tensor(opt.state[a][key]) and opt.state[a][key].numel() == a.numel():
                G.assert_bits_equal(opt.state[a][key], twin.state[b][key], f"{case} {key} {i}")


def test_step_with_a_closure(hip_device):
    """``step(closure)`` re-evaluates the model with gradients enabled, steps on the gradients the
    closure produced and returns its loss (optimi/adam.py:152-155)."""
    model, params = make(torch.bfloat16, hip_device, seed=5)
    opt = optimi_amd.AdamW(params, lr=1e-3)
    ref = oracle_for("adamw", params, dict(lr=1e-3))
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(16, 128, generator=gen).to(torch.bfloat16).to(hip_device)
    y = torch.randn(16, 1, generator=gen).to(torch.bfloat16).to(hip_device)
    calls = []

    def closure():
        opt.zero_grad()
        loss = torch.nn.functional.mse_loss(model(x), y)
        loss.backward()
        calls.append(torch.is_grad_enabled())
        return loss

    for _ in range(3):
        loss = opt.step(closure)
        assert loss is not None and loss.requires_grad and calls[-1] is True
        ref.step([p.grad.detach().cpu().clone() for p in params])
    compare(opt, params, ref, "closure")


@pytest.mark.parametrize("case", ["adamw", "stableadamw", "lion"])
def test_parameters_that_are_views_into_a_flat_buffer(case, hip_device):
    """Parameters carved out of one flat buffer (flattened-parameter wrappers do this) start wherever
    the previous one ended, so most are not 16-byte aligned while their freshly allocated states and
    gradients are: the kernels take the element-wise path for such a tensor and must not touch its
    neighbours in the buffer."""
    cls, oname, hyper = CASES[case]
    gen = torch.Generator().manual_seed(41)
    sizes = [1001, 8195, 3, 4099, 70000]
    for dtype in (torch.bfloat16, torch.float32):
        flat = torch.full((sum(sizes) + 2 * len(sizes) + 9,), 7.0, dtype=dtype, device=hip_device)
        params, spans, at = [], [], 1  # one element in: even the first view is off the 16-byte grid
        for n in sizes:
            view = flat[at:at + n]
            view.copy_((torch.randn(n, generator=gen) * 0.02).to(dtype))
            params.append(torch.nn.Parameter(view))
            spans.append((at, at + n))
            at += n + 2  # two untouched elements between neighbours
        assert any(p.data_ptr() % 16 for p in params)
        opt = cls(params, **hyper)
        ref = oracle_for(oname, params, hyper)
        for _ in range(4):
            for p in params:
                p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(dtype).to(hip_device)
            ref.step([p.grad.detach().cpu().clone() for p in params])
            opt.step()
            opt.zero_grad()
        compare(opt, params, ref, f"{case} {dtype} views")
        keep = torch.ones_like(flat, dtype=torch.bool)
        for a, b in spans:
            keep[a:b] = False
        assert bool((flat[keep] == 7.0).all()), "wrote between the views"


@pytest.mark.parametrize("case", ["adamw", "stableadamw", "adan"])
def test_dense_parameter_with_permuted_strides(case, hip_device):
    """A parameter that is dense in memory but not contiguous (a transposed weight, a
    channels-last filter): its states are created with the same strides (``zeros_like`` with
    ``preserve_format``), its gradient is brought to them, and the step is element-wise, so the
    result equals the oracle's on the logical tensor."""
    cls, oname, hyper = CASES[case]
    gen = torch.Generator().manual_seed(23)
    for dtype in (torch.bfloat16, torch.float32):
        w = torch.nn.Parameter((torch.randn(96, 130, generator=gen) * 0.02).to(dtype).to(hip_device).t())
        f = torch.nn.Parameter((torch.randn(6, 5, 7, 3, generator=gen) * 0.02).to(dtype).to(hip_device)
                               .contiguous(memory_format=torch.channels_last))
        assert not w.is_contiguous() and not f.is_contiguous()
        params = [w, f]
        opt = cls(params, **hyper)
        ref = oracle_for(oname, params, hyper)
        for step in range(4):
            for p in params:
                g = (torch.randn(p.shape, generator=gen) * 1e-3).to(dtype).to(hip_device)  # contiguous: other strides than p
                p.grad = g if step % 2 else torch.empty_like(p).copy_(g)  # on even steps already in p's layout
            ref.step([p.grad.detach().cpu().contiguous() for p in params])
            opt.step()
            opt.zero_grad()
        assert opt.state[w]["exp_avg"].stride() == w.stride() and opt.state[f]["exp_avg"].stride() == f.stride()
        compare(opt, params, ref, f"{case} {dtype} permuted")


def test_two_optimizers_stepping_from_two_threads(hip_device):
    """Two optimizers, each driven by its own Python thread on its own stream: every launch uses
    the calling thread's current stream and the optimizer's own launch workspace, so the threads
    do not disturb each other (20 tensors each: device tables; StableAdamW: reduction scratch)."""
    import threading

    shapes = [(300, 70), (8200,), (5,), (4096, 16), (513,)] * 4
    results, errors = {}, []

    def work(name, seed):
        try:
            cls, oname, hyper = CASES[name]
            gen = torch.Generator().manual_seed(seed)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).bfloat16().to(hip_device)) for s in shapes]
                opt = cls(params, **hyper)
                ref = oracle_for(oname, params, hyper)
                for _ in range(6):
                    grads = [(torch.randn(s, generator=gen) * 1e-3).bfloat16() for s in shapes]
                    for p, g in zip(params, grads):
                        p.grad = g.to(hip_device)
                    opt.step()
                    ref.step(grads)
                stream.synchronize()
            results[name] = (opt, params, ref)
        except Exception as exc:  # noqa: BLE001 - reported by the main thread
            errors.append((name, exc))

    threads = [threading.Thread(target=work, args=(n, i)) for i, n in enumerate(["adamw", "stableadamw"])]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for name, (opt, params, ref) in results.items():
        compare(opt, params, ref, f"threaded {name}")


@pytest.mark.parametrize("release", [False, True], ids=["step", "gradient_release"])
def test_a_tensor_learning_rate_filled_in_place_is_seen(release, hip_device):
    """torch's schedulers fill a tensor learning rate in place (``param_group["lr"].fill_(x)``): the group
    dict is not modified then, so the native drivers, which reuse a group's step scalars while its dict is
    unmodified, must not reuse them for values that can change underneath it.  An optimizer whose lr is a
    float64 tensor, filled in place between steps, against one that is handed plain floats."""
    gen = torch.Generator().manual_seed(41)
    shapes = [(40, 30), (8200,), (64,)] * 6
    start = [(torch.randn(s, generator=gen) * 0.02).to(torch.bfloat16).to(hip_device) for s in shapes]
    models = []
    for lr in (torch.tensor(1e-3, dtype=torch.float64), 1e-3):
        model = torch.nn.Module()
        model.ps = torch.nn.ParameterList([torch.nn.Parameter(p.clone()) for p in start])
        opt = optimi_amd.AdamW(model.parameters(), lr=lr, weight_decay=1e-2, gradient_release=release)
        if release:
            optimi_amd.prepare_for_gradient_release(model, opt)
        models.append((model, opt))
    lrs = [1e-3, 1e-3, 5e-4, 5e-4, 2.5e-4, 1e-3]
    for it, lr in enumerate(lrs):
        models[0][1].param_groups[0]["lr"].fill_(lr)   # in place: the dict keeps the same tensor object
        models[1][1].param_groups[0]["lr"] = lr
        grads = [(torch.randn(s, generator=gen) * 1e-3).to(torch.bfloat16).to(hip_device) for s in shapes]
        for model, opt in models:
            if release:
                loss = sum((p * g).sum() for p, g in zip(model.ps, grads))
                loss.backward()
            else:
                for p, g in zip(model.ps, grads):
                    p.grad = g.clone()
                opt.step()
                opt.zero_grad()
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(models[0][0].ps, models[1][0].ps)):
        G.assert_bits_equal(a, b, f"param {i}")
        for key in ("exp_avg", "exp_avg_sq", "kahan_comp"):
            G.assert_bits_equal(models[0][1].state[a][key], models[1][1].state[b][key], f"{key} {i}")
    for model, _ in models:
        if release:
            optimi_amd.remove_gradient_release(model)
