"""Parity at the sizes of the benchmark configurations.

* C2 – AdamW bf16 + Kahan, ``decouple_lr``, wd 1e-5, the whole Llama-1B-shaped list (147 tensors,
  1,204,881,408 params), 10 steps with fresh gradients: every tensor against the C emulator, bit-exact.
* headline – AdamW bf16 + Kahan on the whole Llama-7B-shaped list (290 tensors, 6,738,411,520 params),
  10 steps with fresh gradients: every tensor, moment and Kahan buffer against the C emulator on the
  host, bit-exact (the result optimi/adam.py:354-396 defines).
* C3/C4 – AdamW, Lion, StableAdamW, Adan in bf16 + Kahan on the same list: the whole list is stepped
  in one launch and every one of its 290 tensors is also stepped through the per-tensor entry point
  from cloned inputs – a whole-list launch must equal per-tensor launches bit for bit, whatever the
  list size.  The five distinct shapes are checked against the C emulator on the CPU (10 steps).
* the same 7B list with fp32 embeddings and norm weights beside bf16 + Kahan (AdamW, StableAdamW): one launch
  over both dtypes equals per-tensor launches bit for bit.
* C5 – AdamW bf16 + Kahan per tensor in reverse order with ``accumulation_steps=4`` on the 7B shapes
  sample, and the 10,000-tensor stress list (sizes log-uniform in [128, 65536]) both as one launch and
  as 10,000 per-tensor launches, against the C emulator.
Gradients are drawn on the GPU (seeded) and copied to the host for the oracle.
"""

import math

import pytest
import torch

import golden_util as G
from oracle.scalar import ScalarRun

pytestmark = pytest.mark.gpu

ADAMW = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
HYPER = {
    "lion": dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1),
    "stableadamw": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2),
    "adan": dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2, kahan_sum=True),
    "adamw": ADAMW,
}


def llama_shapes(hidden, inter, layers, vocab=32000, final_norm=False):
    shapes = [(vocab, hidden)]
    for _ in range(layers):
        shapes += [(hidden, hidden)] * 4 + [(inter, hidden)] * 2 + [(hidden, inter)] + [(hidden,)] * 2
    if final_norm:
        shapes.append((hidden,))
    shapes.append((vocab, hidden))
    return shapes


def draw(shapes, device, gen, std, ones_for_1d=False):
    out = []
    for s in shapes:
        if ones_for_1d and len(s) == 1:
            out.append(torch.ones(s, dtype=torch.bfloat16, device=device))
        else:
            out.append(torch.empty(s, dtype=torch.float32, device=device).normal_(0, std, generator=gen).bfloat16())
    return out


def free():
    import gc

    gc.collect()
    torch.cuda.empty_cache()


def test_c2_adamw_llama1b_whole_list(hip_device):
    from hip_engine import HipRun

    shapes = llama_shapes(2048, 8192, 16, final_norm=True)
    assert len(shapes) == 147 and sum(math.prod(s) for s in shapes) == 1_204_881_408
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-5, decouple_lr=True)
    gen = torch.Generator(device=hip_device).manual_seed(2)
    params = draw(shapes, hip_device, gen, 0.02, ones_for_1d=True)
    hip = HipRun("adamw", params, **hyper)
    sca = ScalarRun("adamw", [p.cpu() for p in params], **hyper)
    for _ in range(10):
        grads = draw(shapes, hip_device, gen, 1e-3)
        hip.step(grads)
        sca.step([g.cpu() for g in grads])
        del grads
    G.compare_engines(hip, sca, "C2", exact=True)
    del hip, sca, params
    free()


@pytest.mark.parametrize("name", ["lion", "stableadamw", "adan", "adamw"])
def test_c3_c4_llama7b_whole_list_equals_per_tensor(name, hip_device):
    from hip_engine import HipRun

    shapes = llama_shapes(4096, 11008, 32)
    assert len(shapes) == 290 and sum(math.prod(s) for s in shapes) == 6_738_411_520
    hyper = HYPER[name]
    gen = torch.Generator(device=hip_device).manual_seed(3)
    params = draw(shapes, hip_device, gen, 0.02, ones_for_1d=True)
    every = list(range(len(shapes)))  # all 290 tensors: both sides live on the GPU (Adan: 2 x 94 GB of the 288)
    sample = HipRun(name, [params[i].clone() for i in every], gradient_release=True, **hyper)  # per-tensor entry points
    whole = HipRun(name, params, **hyper)
    for _ in range(2):
        grads = draw(shapes, hip_device, gen, 1e-3)
        for j, i in enumerate(every):
            sample.step_param(j, grads[i])
        whole.step(grads)
        del grads
    torch.cuda.synchronize()
    for j, i in enumerate(every):
        assert bits_equal_on_device(whole.params[i], sample.params[j]), f"{name} tensor {i} param"
        for key in G.STATE_KEYS:
            a = whole.state[i].get(key)
            if a is not None:
                assert bits_equal_on_device(a, sample.state[j][key]), f"{name} tensor {i} {key}"
    del whole, sample, params
    free()


def bits_equal_on_device(a, b):
    """Bit equality of two device tensors without a trip to the host (a NaN's sign and payload are free)."""
    view = torch.int16 if a.dtype in (torch.bfloat16, torch.float16) else torch.int32
    bad = (a.view(view) != b.view(view)) & ~(torch.isnan(a) & torch.isnan(b))
    return not bool(bad.any())


@pytest.mark.parametrize("name", ["adamw", "stableadamw"])
def test_llama7b_list_of_mixed_dtypes_equals_per_tensor(name, hip_device):
    """The 7B list with its embeddings and norm weights in fp32 (262 M parameters, two of the tensors
    past 2^27 elements) beside bf16 + Kahan: one launch over both dtypes against per-tensor launches
    of each tensor's own dtype, bit for bit - 13.7 M workgroups, chunks of 8192 and of 4096 elements
    in one grid."""
    from hip_engine import HipRun

    from optimi_amd import cabi

    shapes = llama_shapes(4096, 11008, 32)
    hyper = HYPER[name]
    gen = torch.Generator(device=hip_device).manual_seed(7)
    params = draw(shapes, hip_device, gen, 0.02, ones_for_1d=True)
    fp32 = [i for i, s in enumerate(shapes) if len(s) == 1 or s[0] == 32000]
    assert len(fp32) == 66 and sum(math.prod(shapes[i]) for i in fp32) == 262_406_144
    for i in fp32:
        params[i] = params[i].float()
    every = list(range(len(shapes)))
    sample = HipRun(name, [params[i].clone() for i in every], gradient_release=True, **hyper)
    whole = HipRun(name, params, **hyper)
    for _ in range(2):
        grads = draw(shapes, hip_device, gen, 1e-3)
        for i in fp32:
            grads[i] = grads[i].float()
        for j, i in enumerate(every):
            sample.step_param(j, grads[i])
        before = cabi.lib().optimi_hip_launch_count()
        whole.step(grads)
        assert cabi.lib().optimi_hip_launch_count() - before == (3 if name == "stableadamw" else 1)
        del grads
    torch.cuda.synchronize()
    assert {p.dtype for p in whole.params} == {torch.bfloat16, torch.float32}
    for j, i in enumerate(every):
        assert bits_equal_on_device(whole.params[i], sample.params[j]), f"{name} tensor {i} param"
        for key in G.STATE_KEYS:
            a = whole.state[i].get(key)
            if a is not None:
                assert bits_equal_on_device(a, sample.state[j][key]), f"{name} tensor {i} {key}"
    del whole, sample, params
    free()


def test_headline_adamw_llama7b_whole_list_against_emulator(hip_device):
    """The workload the headline figure is quoted on, at full size, against the oracle: ten whole-list
    steps of bf16 AdamW with Kahan summation over all 6,738,411,520 parameters, fresh gradients every
    step, then every parameter, moment and Kahan buffer of every tensor compared bit for bit with the C
    emulator, which steps the same inputs on the host (about 81 GB of host memory: five arrays and one
    set of gradients)."""
    import psutil
    from hip_engine import HipRun

    if psutil.virtual_memory().available < 100e9:
        pytest.skip("the host copy of the 6.7 B-parameter list and its states needs about 81 GB of free host memory")
    shapes = llama_shapes(4096, 11008, 32)
    assert len(shapes) == 290 and sum(math.prod(s) for s in shapes) == 6_738_411_520
    gen = torch.Generator(device=hip_device).manual_seed(11)
    params = draw(shapes, hip_device, gen, 0.02, ones_for_1d=True)
    hip = HipRun("adamw", params, **ADAMW)
    sca = ScalarRun("adamw", [p.cpu() for p in params], **ADAMW)
    # the gradients travel to the host through one pinned buffer (13.5 GB): a pageable copy of each tensor is five times slower
    stage = torch.empty(sum(math.prod(s) for s in shapes), dtype=torch.bfloat16, pin_memory=True)
    offsets = [0]
    for s in shapes:
        offsets.append(offsets[-1] + math.prod(s))
    host_grads = [stage[a:b].view(s) for a, b, s in zip(offsets, offsets[1:], shapes)]
    for _ in range(10):
        grads = draw(shapes, hip_device, gen, 1e-3)
        hip.step(grads)
        for h, g in zip(host_grads, grads):
            h.copy_(g, non_blocking=True)
        torch.cuda.synchronize()
        sca.step(host_grads)  # the emulator reads the gradients and leaves them as they are
        del grads
    torch.cuda.synchronize()
    # compared on the device, tensor by tensor: the oracle's result travels up, 5 x 13.5 GB in all
    for i, p in enumerate(hip.params):
        assert bits_equal_on_device(p, sca.params[i].to(hip_device)), f"headline tensor {i} {shapes[i]} param"
        for key in ("exp_avg", "exp_avg_sq", "kahan_comp"):
            assert bits_equal_on_device(hip.state[i][key], sca.state[i][key].to(hip_device)), f"headline tensor {i} {shapes[i]} {key}"
    del hip, sca, params
    free()


DISTINCT_7B = [(32000, 4096), (4096, 4096), (11008, 4096), (4096, 11008), (4096,)]


@pytest.mark.parametrize("name", ["adamw", "lion", "stableadamw", "adan"])
def test_c3_c4_distinct_7b_shapes_against_emulator(name, hip_device):
    from hip_engine import HipRun

    hyper = HYPER[name]
    gen = torch.Generator(device=hip_device).manual_seed(4)
    params = draw(DISTINCT_7B, hip_device, gen, 0.02, ones_for_1d=True)
    hip = HipRun(name, params, **hyper)
    sca = ScalarRun(name, [p.cpu() for p in params], **hyper)
    for _ in range(10):
        grads = draw(DISTINCT_7B, hip_device, gen, 1e-3)
        hip.step(grads)
        sca.step([g.cpu() for g in grads])
    G.compare_engines(hip, sca, f"{name} 7B shapes", exact=name != "stableadamw")
    del hip, sca, params
    free()


def test_c5_release_with_accumulation_7b_shapes(hip_device):
    from hip_engine import HipRun

    gen = torch.Generator(device=hip_device).manual_seed(5)
    params = draw(DISTINCT_7B, hip_device, gen, 0.02, ones_for_1d=True)
    hip = HipRun("adamw", params, gradient_release=True, **ADAMW)
    sca = ScalarRun("adamw", [p.cpu() for p in params], gradient_release=True, **ADAMW)
    for t in range(8):
        hip.optimizer_accumulation = sca.optimizer_accumulation = (t + 1) % 4 != 0
        grads = draw(DISTINCT_7B, hip_device, gen, 1e-3)
        for i in reversed(range(len(params))):
            hip.step_param(i, grads[i])
            sca.step_param(i, grads[i].cpu())
    G.compare_engines(hip, sca, "C5 release", exact=True)
    del hip, sca, params
    free()


def test_c5_stress_list_10000_tensors(hip_device):
    from hip_engine import HipRun

    rng = torch.Generator().manual_seed(6)
    sizes = torch.exp(torch.empty(10_000).uniform_(math.log(128), math.log(65536), generator=rng)).long().clamp(128, 65536).tolist()
    assert len(sizes) == 10_000 and 0.8e8 < sum(sizes) < 1.3e8
    shapes = [(n,) for n in sizes]
    gen = torch.Generator(device=hip_device).manual_seed(7)
    params = draw(shapes, hip_device, gen, 0.02)
    multi = HipRun("adamw", [p.clone() for p in params], **ADAMW)
    single = HipRun("adamw", [p.clone() for p in params], gradient_release=True, **ADAMW)
    sca = ScalarRun("adamw", [p.cpu() for p in params], **ADAMW)
    for _ in range(3):
        grads = draw(shapes, hip_device, gen, 1e-3)
        multi.step(grads)
        for i in reversed(range(len(shapes))):
            single.step_param(i, grads[i])
        sca.step([g.cpu() for g in grads])
    G.compare_engines(multi, sca, "stress multi", exact=True)
    G.compare_engines(single, multi, "stress per-tensor", exact=True)
    del multi, single, sca, params
    free()
