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


def textbook(name, params, grads, *, lr, betas, eps=0.0, wd=0.0):
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
