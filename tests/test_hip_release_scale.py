"""Gradient release through the product's own machinery at the sizes of the benchmark's fifth
configuration: ``prepare_for_gradient_release`` installs the native post-accumulate-grad hook on
real ``nn.Parameter``s, an autograd function hands each backward pass a fresh set of gradients,
the hook parks small tensors in the coalescing queue and launches large ones at once, and the
autograd engine's final callback flushes what is still parked.  ``accumulation_steps = 4``
(three accumulate-only passes, then a full step), 8 passes.

* the 10,000-tensor stress list (sizes log-uniform in [128, 65536] elements): every tensor,
  every state, bit for bit against the C emulator stepping per tensor on the CPU; the queue's
  tensor and element limits must both have been hit on every pass;
* the Llama-7B-shaped list (290 tensors): all of it stepped by the hooks, a sample that covers
  every distinct shape checked bit for bit against the C emulator.

Follows optimi/gradientrelease.py:13-45 and optimi/adam.py:183-208.
"""

import math

import pytest
import torch

import golden_util as G
import optimi_amd
from oracle.scalar import ScalarRun

pytestmark = pytest.mark.gpu

ADAMW = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
PASSES = 8


def make_feed(current):
    """An autograd function whose backward hands ``current[0]`` (a list of gradients, one per
    parameter) to the parameters: a backward pass that launches no kernels of its own."""

    class Feed(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *ps):
            return ps[0].new_zeros(())

        @staticmethod
        def backward(ctx, grad_out):
            return tuple(g.view(g.shape) for g in current[0])  # fresh tensor objects, adopted as .grad

    return Feed


def draw(shapes, device, gen, std, ones_for_1d=False):
    out = []
    for s in shapes:
        if ones_for_1d and len(s) == 1:
            out.append(torch.ones(s, dtype=torch.bfloat16, device=device))
        else:
            out.append(torch.empty(s, dtype=torch.float32, device=device).normal_(0, std, generator=gen).bfloat16())
    return out


def check_against(opt, params, sca, idxs, what):
    for j, i in enumerate(idxs):
        p, st, ref = params[i], opt.state[params[i]], sca.state[j]
        G.assert_bits_equal(p.detach(), sca.params[j], f"{what} tensor {i} param")
        for key in ("exp_avg", "exp_avg_sq", "kahan_comp"):
            G.assert_bits_equal(st[key], ref[key], f"{what} tensor {i} {key}")
        assert int(st["step"]) == int(ref["step"]) == PASSES
        assert p.grad is None


@pytest.mark.parametrize("max_bytes", [None, 8 << 20], ids=["default_limits", "byte_limit_8M"])
def test_hooks_on_the_10000_tensor_stress_list(max_bytes, hip_device):
    """With the default limits the queue launches every 1024 parked tensors (a pass parks more
    than ``_QUEUE_MAX_BYTES`` of gradients in all, but 1024 average tensors stay below it); with
    the byte limit lowered to 8 MiB that limit cuts every launch short instead."""
    rng = torch.Generator().manual_seed(6)
    sizes = torch.exp(torch.empty(10_000).uniform_(math.log(128), math.log(65536), generator=rng)).long().clamp(128, 65536).tolist()
    shapes = [(n,) for n in sizes]
    gen = torch.Generator(device=hip_device).manual_seed(8)
    params = [torch.nn.Parameter(p) for p in draw(shapes, hip_device, gen, 0.02)]
    model = torch.nn.Module()
    model.ps = torch.nn.ParameterList(params)
    opt = optimi_amd.AdamW(params, gradient_release=True, **ADAMW)
    if max_bytes is not None:
        opt._QUEUE_MAX_BYTES = max_bytes
    optimi_amd.prepare_for_gradient_release(model, opt)
    assert 2 * sum(sizes) > opt._QUEUE_MAX_BYTES and max(sizes) <= opt.gradient_release_coalesce
    by_tensor_limit = math.ceil(len(params) / opt._QUEUE_MAX_TENSORS)

    sca = ScalarRun("adamw", [p.detach().cpu() for p in params], gradient_release=True, **ADAMW)
    current = [None]
    feed = make_feed(current)
    queue = opt._queue()
    for t in range(PASSES):
        accumulate = (t + 1) % 4 != 0
        opt.optimizer_accumulation = sca.optimizer_accumulation = accumulate
        current[0] = draw(shapes, hip_device, gen, 1e-3)
        before, steps_before = queue.launches(), queue.launched_steps()
        feed.apply(*params).backward()
        # every tensor is small enough to be parked: all 10,000 steps went through list launches,
        # at least ten of them (1024 tensors each at most)
        assert queue.pending() == 0
        assert queue.launched_steps() - steps_before == len(params)
        flushes = queue.launches() - before
        assert flushes >= by_tensor_limit == 10, flushes
        if max_bytes is not None:  # about 210 MB of gradients per pass, at most 8 MiB + one tensor per launch
            assert flushes >= 2 * sum(sizes) // (max_bytes + 2 * 65536) > 2 * by_tensor_limit, flushes
        for i in reversed(range(len(params))):  # the order autograd releases them in does not matter: steps are per tensor
            sca.step_param(i, current[0][i].cpu())
    torch.cuda.synchronize()
    check_against(opt, params, sca, range(len(params)), "stress list")
    optimi_amd.remove_gradient_release(model)


def llama_shapes(hidden, inter, layers, vocab=32000):
    shapes = [(vocab, hidden)]
    for _ in range(layers):
        shapes += [(hidden, hidden)] * 4 + [(inter, hidden)] * 2 + [(hidden, inter)] + [(hidden,)] * 2
    shapes.append((vocab, hidden))
    return shapes


SAMPLE_7B = [1, 5, 7, 8, 9, 280, 288, 289]  # q, gate, down, both norms of layer 0; q and a norm of layer 31; lm_head


def test_hooks_on_the_llama7b_list(hip_device):
    import gc

    shapes = llama_shapes(4096, 11008, 32)
    assert len(shapes) == 290 and sum(math.prod(s) for s in shapes) == 6_738_411_520
    gen = torch.Generator(device=hip_device).manual_seed(9)
    params = [torch.nn.Parameter(p) for p in draw(shapes, hip_device, gen, 0.02, ones_for_1d=True)]
    model = torch.nn.Module()
    model.ps = torch.nn.ParameterList(params)
    opt = optimi_amd.AdamW(params, gradient_release=True, **ADAMW)
    optimi_amd.prepare_for_gradient_release(model, opt)
    sca = ScalarRun("adamw", [params[i].detach().cpu() for i in SAMPLE_7B], gradient_release=True, **ADAMW)
    current = [None]
    feed = make_feed(current)
    queue = opt._queue()
    n_small = sum(1 for s in shapes if math.prod(s) <= opt.gradient_release_coalesce)
    assert n_small == 288  # everything but the embedding and the output matrix is parked, those two launch from their hooks
    for t in range(PASSES):
        accumulate = (t + 1) % 4 != 0
        opt.optimizer_accumulation = sca.optimizer_accumulation = accumulate
        current[0] = None
        current[0] = draw(shapes, hip_device, gen, 1e-3)
        steps_before = queue.launched_steps()
        feed.apply(*params).backward()
        assert queue.pending() == 0 and queue.launched_steps() - steps_before == n_small
        for j, i in enumerate(SAMPLE_7B):
            sca.step_param(j, current[0][i].cpu())
    torch.cuda.synchronize()
    check_against(opt, params, sca, SAMPLE_7B, "7B list")
    # nothing outside the sample was left behind
    assert all(int(opt.state[p]["step"]) == PASSES and p.grad is None for p in params)
    optimi_amd.remove_gradient_release(model)
    del opt, sca, params, model, current
    gc.collect()
    torch.cuda.empty_cache()
