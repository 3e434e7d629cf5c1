"""Both oracles against the golden vectors written by the reference (tests/golden/*.npz).

* ``oracle.forloop.ForLoopRun`` (same torch ops, same order) must reproduce every snapshot
  bit for bit: it runs the reference's arithmetic on the reference's inputs.
* ``oracle.scalar.ScalarRun`` (hand-written rounding points in C) must be bit-exact on bf16
  tensors and on fp32 moment states.  fp32 parameters may differ in the last bits because
  torch's CPU sqrt is faithfully, not correctly, rounded, and StableAdamW's mean is summed in
  another order: there the bar is |a-b| <= 1e-6 * max(|a|, |b|, 1e-2) (Ranger's slow weights
  are parameters in this sense).  For the optimizers that go through ``add_(x, alpha=...)`` in
  bf16 the last ``numel % 32`` elements are left out (see ``golden_util.torch_tail``).
"""

import pytest
import torch

import golden_util as G
from oracle.forloop import ForLoopRun
from oracle.scalar import ScalarRun


def bits(t):
    return t.contiguous().view(torch.int16 if t.dtype in (torch.bfloat16, torch.float16) else torch.int32)


@pytest.mark.parametrize("name", G.case_names())
def test_forloop_restatement_is_bit_exact(name):
    torch.set_num_threads(1)
    fx = G.load(name)
    out = G.replay(name, fx, ForLoopRun)
    wanted = sorted(k for k in fx if k.startswith("out."))
    assert sorted(out) == wanted
    for k in wanted:
        assert torch.equal(bits(out[k]), bits(fx[k])), f"{name} {k}"


@pytest.mark.parametrize("name", G.case_names())
def test_scalar_emulator(name):
    fx = G.load(name)
    out = G.replay(name, fx, ScalarRun)
    wanted = sorted(k for k in fx if k.startswith("out."))
    assert sorted(out) == wanted
    for k in wanted:
        got, want = out[k].flatten(), fx[k].flatten()
        keep = want.numel() - G.torch_tail(name, want.numel(), want.dtype)
        got, want = got[:keep], want[:keep]
        if want.dtype != torch.float32 or not (".param." in k or ".la_param." in k):
            n_bad = int(((bits(got) != bits(want)) & ~(got.isnan() & want.isnan())).sum())
            assert n_bad == 0, f"{name} {k}: {n_bad} elements differ"
        else:
            rel = G.fp32_rel_err(got, want, 1e-2)
            assert float(rel.max()) <= 1e-6, f"{name} {k}: rel err {float(rel.max())}"


@pytest.mark.parametrize("name", G.case_names())
def test_committed_recipe_regenerates_the_fixture_inputs(name):
    """``make_fixtures.make_inputs`` with the frozen seed of the case reproduces every stored
    ``in.*`` array, so the committed script and the committed files belong together (the outputs
    need the reference; the inputs do not)."""
    _cls, _kwargs, dtype_name, _mode, n_steps = G.CASES[name]
    fx = G.load(name)
    params, grads = G.make_inputs(G.case_dtypes(dtype_name), n_steps, G.SEEDS[name])
    stored = sorted(k for k in fx if k.startswith("in."))
    assert len(stored) == len(params) * (1 + n_steps)
    for i, p in enumerate(params):
        assert torch.equal(bits(p), bits(fx[f"in.param.{i}"])), f"{name} in.param.{i}"
    for t, gs in enumerate(grads):
        for i, g in enumerate(gs):
            assert torch.equal(bits(g), bits(fx[f"in.grad.{t}.{i}"])), f"{name} in.grad.{t}.{i}"
