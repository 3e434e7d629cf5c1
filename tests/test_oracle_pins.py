"""Checks that pin the oracle to something other than its own formulas.

The golden fixtures (test_oracle_golden.py) pin op order and rounding.  The tests here pin
the mathematics: library optimizers that are algebraically the same, the textbook statement
of each algorithm evaluated in float64 with raw moving averages and explicit bias
corrections (the oracle folds the correction into the betas instead), closed forms at the
first step, and invariants of the accumulate-only step and of Kahan summation.  A dropped
term, a wrong sign or a swapped beta fails at least one of them.
"""

import math

import numpy as np
import pytest
import torch

from oracle.forloop import ForLoopRun, debias_beta
from oracle.scalar import ScalarRun

ENGINES = [ForLoopRun, ScalarRun]
SHAPES = [(37, 19), (256,), (5,)]


def draw(seed, dtype=torch.float32, steps=10, scale=1e-3):
    gen = torch.Generator().manual_seed(seed)
    params = [(torch.randn(s, generator=gen) * 0.02).to(dtype) for s in SHAPES]
    grads = [[(torch.randn(s, generator=gen) * scale * (1 + 3 * (t % 3 == 2))).to(dtype) for s in SHAPES] for t in range(steps)]
    return params, grads


def run(engine, name, params, grads, **hyper):
    eng = engine(name, [p.clone() for p in params], **hyper)
    for gs in grads:
        eng.step([g.clone() for g in gs])
    return eng


def test_debias_beta_closed_form():
    for beta in (0.9, 0.92, 0.98, 0.99, 0.999):
        assert debias_beta(beta, 1) == 0.0
        for t in (2, 3, 10, 1000):
            want = beta * (1 - beta ** (t - 1)) / (1 - beta**t)
            assert math.isclose(debias_beta(beta, t), want, rel_tol=1e-12)
        # a debiased EMA with this beta equals the raw EMA divided by (1 - beta^t)
        xs = np.random.default_rng(0).normal(size=20)
        raw, deb = 0.0, 0.0
        for t, x in enumerate(xs, 1):
            raw = beta * raw + (1 - beta) * x
            bh = debias_beta(beta, t)
            deb = bh * deb + (1 - bh) * x
            assert math.isclose(deb, raw / (1 - beta**t), rel_tol=1e-9, abs_tol=1e-12)


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("decoupled", [True, False])
def test_adam_equals_torch_optim(engine, decoupled):
    """fp32 Adam/AdamW is torch.optim.Adam/AdamW up to rounding (the reference's own test,
    tests/opt_adam.py:19-26, opt_adamw.py:19-26, at its tolerance atol 1e-6 / rtol 1e-5)."""
    lr, betas, eps, wd = 1e-3, (0.9, 0.99), 1e-6, 1e-2
    params, grads = draw(1)
    eng = run(engine, "adamw" if decoupled else "adam", params, grads, lr=lr, betas=betas, eps=eps, weight_decay=wd,
              **({} if decoupled else {"decouple_wd": False}))
    tp = [torch.nn.Parameter(p.clone()) for p in params]
    cls = torch.optim.AdamW if decoupled else torch.optim.Adam
    topt = cls(tp, lr=lr, betas=betas, eps=eps, weight_decay=wd, foreach=False)
    for gs in grads:
        for p, g in zip(tp, gs):
            p.grad = g.clone()
        topt.step()
    t = len(grads)
    for i, p in enumerate(tp):
        torch.testing.assert_close(eng.params[i], p.detach(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(eng.state[i]["exp_avg"], topt.state[p]["exp_avg"] / (1 - betas[0] ** t), rtol=1e-5, atol=1e-9)
        torch.testing.assert_close(eng.state[i]["exp_avg_sq"], topt.state[p]["exp_avg_sq"] / (1 - betas[1] ** t), rtol=1e-5, atol=1e-12)


@pytest.mark.parametrize("engine", ENGINES)
def test_fully_decoupled_lr_equals_rescaled_adamw(engine):
    """decouple_lr with lr == max_lr decays by wd, i.e. torch AdamW with weight_decay = wd / lr."""
    lr, wd = 1e-3, 1e-5
    params, grads = draw(2)
    eng = run(engine, "adamw", params, grads, lr=lr, betas=(0.9, 0.99), eps=1e-6, weight_decay=wd, decouple_lr=True)
    tp = [torch.nn.Parameter(p.clone()) for p in params]
    topt = torch.optim.AdamW(tp, lr=lr, betas=(0.9, 0.99), eps=1e-6, weight_decay=wd / lr, foreach=False)
    for gs in grads:
        for p, g in zip(tp, gs):
            p.grad = g.clone()
        topt.step()
    for i, p in enumerate(tp):
        torch.testing.assert_close(eng.params[i], p.detach(), rtol=1e-5, atol=1e-6)


def textbook(name, params, grads, *, lr, betas, eps=0.0, wd=0.0, adam_wd=False):
    """float64, raw EMAs, explicit bias corrections."""
    out = []
    for i, p0 in enumerate(params):
        p = p0.double().numpy().copy()
        m = np.zeros_like(p); v = np.zeros_like(p); d = np.zeros_like(p); prev = None
        for t, gs in enumerate(grads, 1):
            g = gs[i].double().numpy()
            if name == "lion":
                b1, b2 = betas
                u = np.sign(b1 * m + (1 - b1) * g)
                p = p * (1 - lr * wd) - lr * u
                m = b2 * m + (1 - b2) * g
            elif name == "stableadamw":
                b1, b2 = betas
                m = b1 * m + (1 - b1) * g; v = b2 * v + (1 - b2) * g * g
                mh, vh = m / (1 - b1**t), v / (1 - b2**t)
                rms = math.sqrt(np.mean(g * g / np.maximum(vh, eps * eps)))
                lrt = lr / max(1.0, rms)
                p = p * (1 - lrt * wd) - lrt * mh / (np.sqrt(vh) + eps)
            elif name == "adan":
                b1, b2, b3 = betas
                diff = np.zeros_like(g) if prev is None else g - prev
                m = b1 * m + (1 - b1) * g
                d = b2 * d + (1 - b2) * diff
                v = b3 * v + (1 - b3) * (g + b2 * diff) ** 2
                mh, dh, vh = m / (1 - b1**t), d / (1 - b2**t), v / (1 - b3**t)
                if adam_wd:  # decay the weights first, Adam style, instead of Adan's division after the step
                    p = p * (1 - lr * wd) - lr * (mh + b2 * dh) / (np.sqrt(vh) + eps)
                else:
                    p = (p - lr * (mh + b2 * dh) / (np.sqrt(vh) + eps)) / (1 + lr * wd)
                prev = g
        out.append(p)
    return out


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("name,hyper", [
    ("lion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)),
    ("stableadamw", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)),
    ("adan", dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2)),
])
def test_matches_textbook_algorithm(engine, name, hyper):
    params, grads = draw(3)
    eng = run(engine, name, params, grads, **hyper)
    want = textbook(name, params, grads, lr=hyper["lr"], betas=hyper["betas"], eps=hyper.get("eps", 0.0), wd=hyper["weight_decay"])
    for i, w in enumerate(want):
        got = eng.params[i].double().numpy()
        bad = np.abs(got - w) > 1e-6 + 1e-5 * np.abs(w)
        # Lion: sign() of a value within rounding of zero may legitimately flip; nothing else may differ
        assert bad.sum() <= (2 if name == "lion" else 0), f"{name} tensor {i}: {bad.sum()} elements off, max {np.abs(got - w).max()}"


@pytest.mark.parametrize("engine", ENGINES)
def test_adan_adam_style_decay_matches_textbook(engine):
    """``adam_wd=True`` reaches the functional form only (``functional=True`` drives the engines that
    way): weights decay by 1 - lr*wd before the step.  A large decay makes the two styles differ
    far beyond the tolerance, so taking the wrong branch fails."""
    hyper = dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=5.0)
    params, grads = draw(14)
    eng = engine("adan", [p.clone() for p in params], functional=True, adam_wd=True, **hyper)
    cls_style = engine("adan", [p.clone() for p in params], adam_wd=True, **hyper)  # as a class: the flag is dropped
    for gs in grads:
        eng.step([g.clone() for g in gs])
        cls_style.step([g.clone() for g in gs])
    for style, e in ((True, eng), (False, cls_style)):
        want = textbook("adan", params, grads, lr=hyper["lr"], betas=hyper["betas"], eps=hyper["eps"], wd=5.0, adam_wd=style)
        for i, w in enumerate(want):
            got = e.params[i].double().numpy()
            assert (np.abs(got - w) <= 1e-6 + 1e-5 * np.abs(w)).all(), f"adam_wd={style} tensor {i}"
    assert not torch.allclose(eng.params[0], cls_style.params[0], rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("variant", ["momentum_l2", "dampening_torch_init", "plain_decoupled"])
def test_sgd_equals_torch_optim(engine, variant):
    """fp32 SGD is torch.optim.SGD up to rounding (the reference's own comparison, tests/opt_sgd.py).
    ``dampening=True`` makes the buffer an EMA, m = momentum*m + (1 - momentum)*g, which is torch's
    ``dampening = momentum`` once the buffer starts from the first gradient (``torch_init``);
    decoupled decay multiplies the parameter by 1 - lr*wd before the step, which for plain SGD is
    torch's L2 decay with the same coefficient up to the lr^2 term - so that variant is checked
    against an explicit float64 recursion instead."""
    lr, mu, wd = 1e-2, 0.9, 1e-2
    params, grads = draw(11)
    tp = [torch.nn.Parameter(p.clone()) for p in params]
    if variant == "momentum_l2":
        eng = run(engine, "sgd", params, grads, lr=lr, momentum=mu, weight_decay=wd)
        topt = torch.optim.SGD(tp, lr=lr, momentum=mu, weight_decay=wd, foreach=False)
    elif variant == "dampening_torch_init":
        eng = run(engine, "sgd", params, grads, lr=lr, momentum=mu, weight_decay=wd, dampening=True, torch_init=True)
        topt = torch.optim.SGD(tp, lr=lr, momentum=mu, dampening=mu, weight_decay=wd, foreach=False)
    else:
        eng = run(engine, "sgd", params, grads, lr=lr, momentum=0.0, weight_decay=wd, decouple_wd=True)
        for i, p0 in enumerate(params):
            p = p0.double()
            for gs in grads:
                p = p * (1 - lr * wd) - lr * gs[i].double()
            torch.testing.assert_close(eng.params[i].double(), p, rtol=1e-5, atol=1e-7)
            assert eng.state[i]["exp_avg"] is None
        return
    for gs in grads:
        for p, g in zip(tp, gs):
            p.grad = g.clone()
        topt.step()
    for i, p in enumerate(tp):
        torch.testing.assert_close(eng.params[i], p.detach(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(eng.state[i]["exp_avg"], topt.state[p]["momentum_buffer"], rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("decoupled", [True, False])
def test_radam_equals_torch_optim(engine, decoupled):
    """fp32 RAdam is torch.optim.RAdam up to rounding and the place of eps (torch adds it to
    sqrt(v) before the bias correction, the reference after: with eps = 1e-12 the two agree far
    below the tolerance).  14 steps at beta2 = 0.99 cover the unrectified steps (t <= 5) and the
    rectified ones.  The debiased moments map to torch's raw ones as for Adam."""
    lr, betas, eps, wd = 1e-3, (0.9, 0.99), 1e-12, 1e-2
    params, grads = draw(12, steps=14)
    eng = run(engine, "radam", params, grads, lr=lr, betas=betas, eps=eps, weight_decay=wd, decouple_wd=decoupled)
    tp = [torch.nn.Parameter(p.clone()) for p in params]
    topt = torch.optim.RAdam(tp, lr=lr, betas=betas, eps=eps, weight_decay=wd, decoupled_weight_decay=decoupled, foreach=False)
    for gs in grads:
        for p, g in zip(tp, gs):
            p.grad = g.clone()
        topt.step()
    t = len(grads)
    for i, p in enumerate(tp):
        torch.testing.assert_close(eng.params[i], p.detach(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(eng.state[i]["exp_avg"], topt.state[p]["exp_avg"] / (1 - betas[0] ** t), rtol=1e-5, atol=1e-9)
        torch.testing.assert_close(eng.state[i]["exp_avg_sq"], topt.state[p]["exp_avg_sq"] / (1 - betas[1] ** t), rtol=1e-5, atol=1e-12)


def lookahead_radam_float64(params, grads, *, lr, betas, eps, wd, k, alpha):
    """Lookahead (Zhang et al. 2019) wrapped around RAdam (Liu et al. 2020) as the two papers state
    them: raw moving averages, explicit bias corrections, the length of the approximated SMA and
    its rectification term, decoupled decay; every k-th step the slow weights move a fraction
    alpha towards the fast ones and the fast weights restart from them.  float64 throughout."""
    b1, b2 = betas
    rho_inf = 2 / (1 - b2) - 1
    out = []
    for i, p0 in enumerate(params):
        fast = p0.double().numpy().copy()
        slow = fast.copy()
        m = np.zeros_like(fast); v = np.zeros_like(fast)
        for t, gs in enumerate(grads, 1):
            g = gs[i].double().numpy()
            fast = fast * (1 - lr * wd)
            m = b1 * m + (1 - b1) * g
            v = b2 * v + (1 - b2) * g * g
            mh = m / (1 - b1**t)
            rho = rho_inf - 2 * t * b2**t / (1 - b2**t)
            if rho > 5:
                rect = math.sqrt((rho - 4) * (rho - 2) * rho_inf / ((rho_inf - 4) * (rho_inf - 2) * rho))
                fast = fast - lr * rect * mh / (np.sqrt(v / (1 - b2**t)) + eps)
            else:
                fast = fast - lr * mh
            if t % k == 0:
                slow = slow + alpha * (fast - slow)
                fast = slow.copy()
        out.append((fast, slow))
    return out


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("k,alpha", [(6, 0.5), (3, 0.8)])
def test_ranger_matches_lookahead_over_radam(engine, k, alpha):
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
    params, grads = draw(13, steps=14)
    eng = run(engine, "ranger", params, grads, k=k, alpha=alpha, **hyper)
    want = lookahead_radam_float64(params, grads, lr=hyper["lr"], betas=hyper["betas"], eps=hyper["eps"],
                                   wd=hyper["weight_decay"], k=k, alpha=alpha)
    for i, (fast, slow) in enumerate(want):
        for what, got, w in (("param", eng.params[i], fast), ("la_param", eng.state[i]["la_param"], slow)):
            got = got.double().numpy()
            bad = np.abs(got - w) > 1e-6 + 1e-5 * np.abs(w)
            assert bad.sum() == 0, f"ranger k={k} tensor {i} {what}: {bad.sum()} elements off, max {np.abs(got - w).max()}"
    # the periodic synchronisation really happened: with k = 3 the parameters differ from plain RAdam's
    radam = run(engine, "radam", params, grads, decouple_wd=True, **hyper)
    assert not torch.equal(radam.params[0], eng.params[0])


@pytest.mark.parametrize("engine", ENGINES)
def test_first_step_closed_forms(engine):
    params, grads = draw(4, steps=1)
    lr, eps, wd = 1e-3, 1e-6, 1e-2
    g = [x.double() for x in grads[0]]
    p0 = [x.double() for x in params]
    e = run(engine, "adamw", params, grads, lr=lr, betas=(0.9, 0.99), eps=eps, weight_decay=wd)
    for i in range(len(params)):
        torch.testing.assert_close(e.params[i].double(), p0[i] * (1 - lr * wd) - lr * g[i] / (g[i].abs() + eps), rtol=1e-6, atol=1e-9)
        assert torch.equal(e.state[i]["exp_avg"], grads[0][i])
        torch.testing.assert_close(e.state[i]["exp_avg_sq"].double(), g[i] ** 2, rtol=1e-6, atol=0)
    e = run(engine, "adan", params, grads, lr=lr, betas=(0.98, 0.92, 0.99), eps=eps, weight_decay=wd)
    for i in range(len(params)):
        torch.testing.assert_close(e.params[i].double(), (p0[i] - lr * g[i] / (g[i].abs() + eps)) / (1 + lr * wd), rtol=1e-6, atol=1e-9)
        assert float(e.state[i]["exp_avg_diff"].abs().max()) == 0.0
        assert torch.equal(e.state[i]["prev_grad"], -grads[0][i])
    # StableAdamW: at t=1 every g^2/max(v, eps^2) is 1 where |g| > eps, so rms <= 1 and the step is AdamW's
    a = run(engine, "adamw", params, grads, lr=lr, betas=(0.9, 0.99), eps=eps, weight_decay=wd)
    s = run(engine, "stableadamw", params, grads, lr=lr, betas=(0.9, 0.99), eps=eps, weight_decay=wd)
    for i in range(len(params)):
        assert torch.equal(a.params[i], s.params[i])
    # Lion without decay moves every parameter with a non-zero gradient by exactly lr
    l = run(engine, "lion", params, grads, lr=1e-4, betas=(0.9, 0.99), weight_decay=0.0)
    for i in range(len(params)):
        moved = (l.params[i].double() - p0[i]).abs()
        torch.testing.assert_close(moved, torch.full_like(moved, 1e-4), rtol=1e-3, atol=0)
        torch.testing.assert_close(l.state[i]["exp_avg"].double(), 0.01 * g[i], rtol=1e-5, atol=1e-12)


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("name,hyper", [
    ("adamw", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)),
    ("lion", dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)),
    ("stableadamw", dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)),
    ("adan", dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2, kahan_sum=True)),
])
def test_accumulate_only_step(engine, name, hyper):
    """update_parameters=False: params and Kahan buffers untouched; moments as in a full step."""
    params, grads = draw(5, dtype=torch.bfloat16, steps=3)
    full = engine(name, [p.clone() for p in params], gradient_release=True, **hyper)
    acc = engine(name, [p.clone() for p in params], gradient_release=True, **hyper)
    for t, gs in enumerate(grads):
        acc.optimizer_accumulation = t == 2
        if t == 2:
            before = [(p.clone(), acc.state[i]["kahan_comp"].clone()) for i, p in enumerate(acc.params)]
        for i in range(len(params)):
            full.step_param(i, gs[i].clone())
            acc.step_param(i, gs[i].clone())
    for i in range(len(params)):
        assert torch.equal(acc.params[i], before[i][0]) and torch.equal(acc.state[i]["kahan_comp"], before[i][1])
        assert not torch.equal(full.params[i], before[i][0])
        for key in ("exp_avg", "exp_avg_sq", "exp_avg_diff", "prev_grad"):
            if key in full.state[i]:
                assert torch.equal(full.state[i][key], acc.state[i][key]), key


@pytest.mark.parametrize("engine", ENGINES)
def test_kahan_tracks_fp32_shadow(engine):
    """bf16 params + Kahan buffer follow an fp32 run of the same optimizer more closely than
    plain bf16 params do (docs/kahan_summation.md:93-115).  The moments are bf16 in both runs, which
    sets the floor of the distance to the fp32 run; Kahan summation must at least halve it."""
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=0.0)
    params, grads = draw(6, dtype=torch.bfloat16, steps=60)
    kahan = run(engine, "adamw", params, grads, **hyper)
    plain = run(engine, "adamw", params, grads, kahan_sum=False, **hyper)
    shadow = run(engine, "adamw", [p.float() for p in params], [[g.float() for g in gs] for gs in grads], **hyper)
    for i in range(len(params)):
        ref = shadow.params[i].double()
        err_k = (kahan.params[i].double() + kahan.state[i]["kahan_comp"].double() - ref).abs().mean()
        err_p = (plain.params[i].double() - ref).abs().mean()
        assert plain.state[i]["kahan_comp"] is None
        assert float(err_k) < 0.5 * float(err_p), (float(err_k), float(err_p))


@pytest.mark.parametrize("engine", ENGINES)
def test_kahan_flag_is_ignored_for_fp32(engine):
    params, grads = draw(7, steps=3)
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
    a = run(engine, "adamw", params, grads, kahan_sum=True, **hyper)
    b = run(engine, "adamw", params, grads, kahan_sum=False, **hyper)
    for i in range(len(params)):
        assert torch.equal(a.params[i], b.params[i])


def test_emulator_rounding_matches_numpy_and_torch():
    """The C emulator's own fp16 / bf16 conversions (round to nearest even, fp16 subnormals,
    overflow to inf) against numpy's float16 and torch's bfloat16 casts."""
    from oracle import scalar

    L = scalar.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.normal(size=20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, size=20000).astype(np.float32),
        np.arange(0, 1 << 16, dtype=np.uint16).view(np.float16).astype(np.float32),  # every fp16 value
        # ties between neighbouring fp16 values, normal and subnormal
        (np.arange(0, 1 << 15, 97, dtype=np.uint16).view(np.float16).astype(np.float64)
         + np.arange(1, (1 << 15) + 1, 97, dtype=np.uint16).view(np.float16).astype(np.float64)).astype(np.float32) / 2,
        np.array([65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0**-25, 2.0**-25 * 1.0001, 2.0**-24, 0.0, -0.0], dtype=np.float32),
    ])
    xs = xs[np.isfinite(xs)]
    with np.errstate(over="ignore"):
        want16 = xs.astype(np.float16).astype(np.float32)
    wantbf = torch.from_numpy(xs).to(torch.bfloat16).float().numpy()
    got16 = np.array([L.optimi_ref_round(float(x), scalar.F16) for x in xs], dtype=np.float32)
    gotbf = np.array([L.optimi_ref_round(float(x), scalar.BF16) for x in xs], dtype=np.float32)
    got32 = np.array([L.optimi_ref_round(float(x), scalar.F32) for x in xs], dtype=np.float32)
    assert np.array_equal(got16.view(np.uint32), want16.view(np.uint32))
    assert np.array_equal(gotbf.view(np.uint32), wantbf.view(np.uint32))
    assert np.array_equal(got32.view(np.uint32), xs.view(np.uint32))
