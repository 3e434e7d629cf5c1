"""Lists that mix fp32 tensors with tensors of one 16-bit dtype: one launch for the whole list
(``optimi_hip_*_multi_mixed``), the bits of the one-dtype launches.

What is compared with what:
* mixed launch vs two one-dtype launches over the 16-bit and the fp32 tensors of the same list:
  bit-identical, every optimizer, bf16 and fp16, Kahan on and off, update and accumulate-only;
* mixed launch vs ``ForLoopRun`` (the torch restatement of the reference's for-loop path, which
  loops over the tensors of a group whatever their dtypes): the tolerance of the one-dtype tests;
* the launch counter: one kernel per step (three for StableAdamW), where the one-dtype entry
  points need two (six).
The reference's own output for a group of mixed dtypes is held by the ``*_mixed_*`` fixtures
(``tests/test_hip_golden.py`` replays them through the same entry points).
"""

import types

import pytest
import torch

import golden_util as G
from oracle.forloop import ForLoopRun
from test_hip_parity import ADD_ALPHA, CONFIGS, OPT_OF, Guarded, draw, hip_engine

pytestmark = pytest.mark.gpu

# sizes below, at and above the vector, the tile and the chunk of either dtype (an fp32 chunk is
# 4096 elements, a 16-bit one 8192), empty tensors at the start, in the middle and at the end
SIZES = [0, 8193, 5, 4096, 4097, 0, 513, 8192, 1, 20001, 1024, 12288, 7, 100003, 64, 0]
F32_AT = {1, 2, 5, 6, 9, 11, 13, 15}  # positions of the fp32 tensors: both kinds begin, end and neighbour each other
# 16 tensors travel as a kernel argument; four more and the list goes through the device tables
MORE_SIZES, MORE_F32_AT = [700, 12288, 0, 33], {17, 19}


def draw_mixed(low, steps, seed, sizes=SIZES, f32_at=F32_AT):
    params, grads = draw(sizes, torch.float32, steps, seed)
    dt = [torch.float32 if i in f32_at else low for i in range(len(sizes))]
    return [p.to(d) for p, d in zip(params, dt)], [[g.to(d) for g, d in zip(gs, dt)] for gs in grads]


def split_view(eng_low, idx_low, eng_f32, idx_f32, n):
    """Two one-dtype engines presented as one engine over the original list."""
    params, state = [None] * n, [None] * n
    for eng, idx in ((eng_low, idx_low), (eng_f32, idx_f32)):
        for j, i in enumerate(idx):
            params[i], state[i] = eng.params[j], eng.state[j]
    return types.SimpleNamespace(params=params, state=state)


def step(eng, grads, accumulate):
    """A whole-list step through the functional form, which - unlike the optimizer classes - takes
    ``optimizer_accumulation`` for lists too (optimi/adam.py:233, 308)."""
    eng._call(list(range(len(grads))), grads, eng.group_step, accumulate)


def launches():
    from optimi_amd import cabi

    return cabi.lib().optimi_hip_launch_count()


@pytest.mark.parametrize("tables", ["kernel_argument", "device"])
@pytest.mark.parametrize("low,kahan", [(torch.bfloat16, None), (torch.bfloat16, False), (torch.float16, None)],
                         ids=["bf16_kahan", "bf16_plain", "fp16_kahan"])
@pytest.mark.parametrize("cfg", list(CONFIGS))
def test_mixed_list_is_one_launch_with_the_bits_of_two(cfg, low, kahan, tables, hip_device):
    hyper = dict(CONFIGS[cfg])
    if kahan is False:
        hyper["kahan_sum"] = False
    name = OPT_OF[cfg]
    steps = 6
    sizes, f32_at = (SIZES, F32_AT) if tables == "kernel_argument" else (SIZES + MORE_SIZES, F32_AT | MORE_F32_AT)
    params, grads = draw_mixed(low, steps, seed=sum(map(ord, cfg)) + 1, sizes=sizes, f32_at=f32_at)
    idx_f32 = sorted(f32_at)
    idx_low = [i for i in range(len(sizes)) if i not in f32_at]
    pick = lambda col, idx: [col[i] for i in idx]  # noqa: E731
    torch.set_num_threads(1)
    guard = Guarded(hip_device)
    mixed = hip_engine(name, params, hip_device, guard, **hyper)
    only_low = hip_engine(name, pick(params, idx_low), hip_device, guard, **hyper)
    # the fp32 tensors of a group whose Kahan flag is on (because of its 16-bit tensors) still take no Kahan branch
    only_f32 = hip_engine(name, pick(params, idx_f32), hip_device, guard, **hyper)
    ref = ForLoopRun(name, [p.clone() for p in params], **hyper)
    per_step = []
    for t, gs in enumerate(grads):
        accumulate = t == 2  # one accumulate-only step in the middle (optimizer accumulation)
        before = launches()
        step(mixed, [guard(g) for g in gs], accumulate)
        per_step.append(launches() - before)
        step(only_low, [guard(g) for g in pick(gs, idx_low)], accumulate)
        step(only_f32, [guard(g) for g in pick(gs, idx_f32)], accumulate)
        step(ref, [g.clone() for g in gs], accumulate)
    torch.cuda.synchronize()
    guard.check()
    plain_sgd_accumulate = 0 if cfg == "sgd_plain" else 1  # nothing to accumulate into without momentum
    for t, n in enumerate(per_step):
        want = (plain_sgd_accumulate if t == 2 else 1) if name != "stableadamw" else (1 if t == 2 else 3)
        assert n == want, f"{cfg} step {t}: {n} kernel launches for the mixed list, expected {want}"
    G.compare_engines(mixed, split_view(only_low, idx_low, only_f32, idx_f32, len(sizes)), f"{cfg} mixed-vs-split", exact=True)
    tail = 32 if cfg in ADD_ALPHA else 0
    G.compare_engines(mixed, ref, f"{cfg} mixed-vs-forloop", exact=False, body_only=tail)


@pytest.mark.parametrize("cfg", ["adamw", "stableadamw", "adan"])
def test_mixed_entry_point_on_a_list_of_one_dtype(cfg, hip_device):
    """Handed a list that holds one dtype, the mixed entry points step it exactly as their
    one-dtype namesakes do (short lists still travel as a kernel argument)."""
    from hip_engine import HipRun

    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    for dtype in (torch.bfloat16, torch.float32):
        params, grads = draw([8193, 0, 700, 12288, 3], dtype, 3, seed=5)
        a = HipRun(name, [p.to(hip_device) for p in params], mixed=True, **hyper)
        b = HipRun(name, [p.to(hip_device) for p in params], **hyper)
        for gs in grads:
            a.step([g.to(hip_device) for g in gs])
            b.step([g.to(hip_device) for g in gs])
        torch.cuda.synchronize()
        G.compare_engines(a, b, f"{cfg} {dtype} mixed entry, one dtype", exact=True)


def test_mixed_list_changes_between_steps(hip_device):
    """The chunk map of a mixed list depends on the dtypes, not only on the sizes: two lists with
    the same sizes and the dtypes swapped, stepped through one group in turn, must each get their own."""
    from hip_engine import HipRun

    hyper = CONFIGS["adamw"]
    sizes = [6000, 6000, 9000, 9000]
    pa, ga = draw(sizes, torch.float32, 4, seed=3)
    dts = [[torch.bfloat16, torch.float32, torch.bfloat16, torch.float32], [torch.float32, torch.bfloat16, torch.float32, torch.bfloat16]]
    engines, refs = [], []
    shared = None
    for dt in dts:
        eng = HipRun("adamw", [p.to(d).to(hip_device) for p, d in zip(pa, dt)], **hyper)
        if shared is None:
            shared = eng.group
        eng.group = shared  # both lists go through the same launch workspace
        engines.append(eng)
        refs.append(HipRun("adamw", [p.to(d).to(hip_device) for p, d in zip(pa, dt)], multi=False, **hyper))
    for gs in ga:
        for eng, ref, dt in zip(engines, refs, dts):
            eng.step([g.to(d).to(hip_device) for g, d in zip(gs, dt)])
            ref.step([g.to(d).to(hip_device) for g, d in zip(gs, dt)])
    torch.cuda.synchronize()
    for k, (eng, ref) in enumerate(zip(engines, refs)):
        G.compare_engines(eng, ref, f"alternating mixed lists, list {k}", exact=True)


def test_mixed_list_rejections(hip_device):
    import ctypes as C

    from optimi_amd import cabi

    L = cabi.lib()
    grp = cabi.Group()
    t = torch.zeros(64, dtype=torch.float32, device=hip_device)
    a = t.data_ptr()
    ptrs = cabi.ptr_array([a, a])
    numel = cabi.i64_array([16, 16])
    tail = (1e-3, 0.1, 0.9, 0.1, 0.99, 1e-6, cabi.UPDATE | cabi.KAHAN, None)
    dts = lambda *v: (C.c_int * len(v))(*v)  # noqa: E731
    assert L.optimi_hip_adam_multi_mixed(grp.handle, 2, ptrs, ptrs, ptrs, ptrs, ptrs, numel, dts(cabi.BF16, cabi.F16), *tail) == -3
    assert L.optimi_hip_adam_multi_mixed(grp.handle, 2, ptrs, ptrs, ptrs, ptrs, ptrs, numel, dts(cabi.BF16, 5), *tail) == -3
    assert L.optimi_hip_adam_multi_mixed(grp.handle, 2, ptrs, ptrs, ptrs, ptrs, ptrs, numel, None, *tail) == -1
    # the Kahan buffer of the fp32 tensor may be missing, that of the bf16 tensor may not
    kahan = cabi.ptr_array([None, a])
    assert L.optimi_hip_adam_multi_mixed(grp.handle, 2, ptrs, ptrs, ptrs, ptrs, kahan, numel, dts(cabi.BF16, cabi.F32), *tail) == -1
    assert L.optimi_hip_adam_multi_mixed(grp.handle, 2, ptrs, ptrs, ptrs, ptrs, kahan, numel, dts(cabi.F32, cabi.BF16), *tail) == 0
    assert L.optimi_hip_adam_multi_mixed(grp.handle, 0, None, None, None, None, None, None, None, *tail) == 0
    torch.cuda.synchronize()


def test_optimizer_steps_a_mixed_group_in_one_launch(hip_device):
    """A bf16 model with fp32 norm weights: each parameter group is one launch per step, on the
    first step (which goes through the Python functional layer) and on the later ones (the native
    group walk) alike."""
    import optimi_amd

    torch.manual_seed(0)
    w = [torch.nn.Parameter((torch.randn(300, 70) * 0.02).to(torch.bfloat16).to(hip_device)) for _ in range(3)]
    n = [torch.nn.Parameter(torch.ones(70, device=hip_device)) for _ in range(4)]
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6)
    order = [w[0], n[0], w[1], n[1], w[2]]
    opt = optimi_amd.AdamW([{"params": order, "weight_decay": 1e-2}, {"params": n[2:], "weight_decay": 0.0}], **hyper)
    ref_decay = ForLoopRun("adamw", [p.detach().cpu().clone() for p in order], weight_decay=1e-2, **hyper)
    ref_plain = ForLoopRun("adamw", [p.detach().cpu().clone() for p in n[2:]], weight_decay=0.0, **hyper)
    gen = torch.Generator().manual_seed(5)
    for t in range(5):
        for p in w + n:
            p.grad = (torch.randn(p.shape, generator=gen) * 1e-3).to(p.dtype).to(hip_device)
        ref_decay.step([p.grad.cpu().clone() for p in order])
        ref_plain.step([p.grad.cpu().clone() for p in n[2:]])
        before = launches()
        opt.step()
        assert launches() - before == 2, f"step {t}: {launches() - before} launches for two parameter groups"
        opt.zero_grad()
    for p, q in zip(order, ref_decay.params):
        G.assert_close_to_reference(p, q, "mixed decay group", is_param=True)
    for p, q in zip(n[2:], ref_plain.params):
        G.assert_close_to_reference(p, q, "fp32 group", is_param=True)


def test_gradient_release_queue_keeps_mixed_tensors_together(hip_device):
    """During gradient release the hooks of a bf16 model with fp32 norms fire in alternation; the
    queue must not break its run at every change of dtype.  One backward pass over 12 small
    tensors of both kinds ends in one launch, with the results of per-tensor launches."""
    import optimi_amd

    torch.manual_seed(1)

    def make():
        torch.manual_seed(1)
        ps = []
        for i in range(12):
            dt = torch.float32 if i % 2 else torch.bfloat16
            ps.append(torch.nn.Parameter((torch.randn(40, 33) * 0.05).to(dt).to(hip_device)))
        return ps

    def loss_of(ps, x):
        y = x
        for p in ps:
            y = y * 0.5 + (p.float() * x).sum() * 1e-3
        return y.sum()

    runs = {}
    for coalesce in (True, False):
        ps = make()
        opt = optimi_amd.AdamW(ps, lr=1e-3, gradient_release=True)
        if not coalesce:
            opt.gradient_release_coalesce = 0
        mod = torch.nn.Module()
        mod.ps = torch.nn.ParameterList(ps)
        optimi_amd.prepare_for_gradient_release(mod, opt)
        per_pass = []
        for t in range(3):
            x = torch.full((40, 33), 0.1 * (t + 1), device=hip_device)
            before = launches()
            loss_of(ps, x).backward()
            opt.step()
            per_pass.append(launches() - before)
        torch.cuda.synchronize()
        runs[coalesce] = ([p.detach().clone() for p in ps], per_pass)
        optimi_amd.remove_gradient_release(mod)
    # the very first hook call of an optimizer goes through the Python path (it resolves the backend) and launches on its own
    assert runs[True][1][0] <= 2 and runs[True][1][1:] == [1, 1], f"launches per backward pass with the queue: {runs[True][1]}"
    assert runs[False][1] == [12, 12, 12]
    for i, (a, b) in enumerate(zip(runs[True][0], runs[False][0])):
        G.assert_bits_equal(a, b, f"queued vs per-tensor release, tensor {i}")
