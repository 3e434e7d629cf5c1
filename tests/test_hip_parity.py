"""HIP kernels against the CPU oracles on seeded random lists, through the C ABI.

What is compared with what:
* HIP vs ``ScalarRun`` (C emulator with hand-written rounding points): bit-exact, fp32 and
  bf16 alike, for Adam/AdamW, Lion and Adan.  StableAdamW sums its per-tensor mean in another
  order, so there the north-star tolerance applies instead.
* HIP vs ``ForLoopRun`` (the torch restatement of the reference's for-loop path): the
  north-star tolerance – bf16 params, states within 1 ulp and Kahan buffers within 1 ulp of
  the parameter; fp32 within rel 1e-6 – after 10 steps.
* whole-list launch vs per-tensor launches: bit-identical.

Shapes cover every path of the kernel: sizes below, at and above the 8-element vector, the
512-element tile and the 8192-element chunk, buffers that are not 16-byte aligned, empty
tensors, and guard bands around every buffer that must stay untouched.
"""

import ctypes

import pytest
import torch

import golden_util as G
from oracle.forloop import ForLoopRun
from oracle.scalar import ScalarRun

pytestmark = pytest.mark.gpu

SIZES = [1, 7, 8, 9, 63, 64, 65, 511, 512, 513, 1000, 4095, 4096, 4097, 8191, 8192, 8193, 16392, 100003]
GUARD = 64  # elements of sentinel on each side of every buffer

CONFIGS = {
    "adamw": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2),
    "adam_l2": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, decouple_wd=False),
    "adamw_declr": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-5, decouple_lr=True),
    "lion": dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1),
    "stableadamw": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2),
    "adan": dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=2e-2, kahan_sum=True),
    "adan_nowd": dict(lr=1e-3, betas=(0.98, 0.92, 0.99), eps=1e-8, weight_decay=0.0),
    "sgd_momentum": dict(lr=1e-2, momentum=0.9, weight_decay=1e-2, decouple_wd=True),
    "sgd_dampening_l2": dict(lr=1e-2, momentum=0.9, weight_decay=1e-2, dampening=True, torch_init=True),
    "sgd_plain": dict(lr=1e-2, momentum=0.0, weight_decay=0.0),
    "radam": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, decouple_wd=True),
    "ranger": dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2, k=3, alpha=0.5),
}
OPT_OF = {"adamw": "adamw", "adam_l2": "adam", "adamw_declr": "adamw", "lion": "lion", "stableadamw": "stableadamw",
          "adan": "adan", "adan_nowd": "adan", "sgd_momentum": "sgd", "sgd_dampening_l2": "sgd", "sgd_plain": "sgd",
          "radam": "radam", "ranger": "ranger"}
# configurations whose bf16 runs go through ATen's add_(x, alpha=...), which is not uniform over a tensor
ADD_ALPHA = {"adam_l2", "sgd_momentum", "sgd_dampening_l2", "sgd_plain", "radam", "ranger"}


def draw(sizes, dtype, steps, seed):
    gen = torch.Generator().manual_seed(seed)
    params = []
    for n in sizes:
        p = torch.randn(n, generator=gen) * 0.02
        if n >= 4:
            p[:4] = torch.tensor([0.0, -0.0, 1.0, -3.0e-5])
        params.append(p.to(dtype))
    grads = []
    for t in range(steps):
        gs = []
        for n in sizes:
            g = torch.randn(n, generator=gen) * 1e-3 * (1.0, 1.0, 4.0, 0.5, 2.0)[t % 5]
            if n >= 8:
                g[:8] = torch.tensor([0.0, -0.0, 1e-9, -1e-9, 1.0, -0.5, 3e-7, 65504.0])
            gs.append(g.to(dtype))
        grads.append(gs)
    return params, grads


class Guarded:
    """Places a tensor inside a larger device buffer filled with a sentinel; ``offset`` shifts it
    by that many elements so its address is not 16-byte aligned."""

    SENTINEL = 1.2345

    def __init__(self, device):
        self.device = device
        self.bufs = []

    def __call__(self, t: torch.Tensor, offset=0):
        n = t.numel()
        buf = torch.full((n + 2 * GUARD + 8,), self.SENTINEL, dtype=t.dtype, device=self.device)
        view = buf[GUARD + offset: GUARD + offset + n]
        view.copy_(t.flatten())
        self.bufs.append((buf, GUARD + offset, n))
        return view

    def check(self):
        s = torch.tensor(self.SENTINEL)
        for buf, start, n in self.bufs:
            want = s.to(buf.dtype).item()
            assert bool((buf[:start] == want).all()) and bool((buf[start + n:] == want).all()), "write outside a buffer"


def hip_engine(name, params, device, guard, offset=0, **kw):
    from hip_engine import HipRun

    eng = HipRun(name, [guard(p, offset) for p in params], **kw)
    ensure = eng._ensure_state

    def ensure_guarded(i, grad):  # states go into guarded buffers too
        fresh = eng.state[i] is None
        st = ensure(i, grad)
        if fresh:
            for k, v in st.items():
                if torch.is_tensor(v) and v.numel() == eng.params[i].numel() and v.is_cuda:
                    st[k] = guard(v, offset)
        return st

    eng._ensure_state = ensure_guarded
    return eng


@pytest.mark.parametrize("dtype,kahan", [(torch.bfloat16, None), (torch.bfloat16, False), (torch.float32, None),
                                         (torch.float16, None), (torch.float16, False)],
                         ids=["bf16_kahan", "bf16_plain", "fp32", "fp16_kahan", "fp16_plain"])
@pytest.mark.parametrize("cfg", list(CONFIGS))
def test_random_lists_match_both_oracles(cfg, dtype, kahan, hip_device):
    hyper = dict(CONFIGS[cfg])
    if kahan is False:
        hyper["kahan_sum"] = False
    name = OPT_OF[cfg]
    params, grads = draw(SIZES, dtype, 10, seed=sum(map(ord, cfg)))
    torch.set_num_threads(1)  # one remainder loop per tensor in the torch oracle, at its very end
    guard = Guarded(hip_device)
    hip = hip_engine(name, params, hip_device, guard, **hyper)
    hip1 = hip_engine(name, params, hip_device, guard, multi=False, **hyper)
    sca = ScalarRun(name, [p.clone() for p in params], **hyper)
    ref = ForLoopRun(name, [p.clone() for p in params], **hyper)
    for gs in grads:
        hip.step([guard(g) for g in gs])
        hip1.step([guard(g) for g in gs])
        sca.step([g.clone() for g in gs])
        ref.step([g.clone() for g in gs])
    torch.cuda.synchronize()
    guard.check()
    G.compare_engines(hip1, hip, f"{cfg} single-vs-multi", exact=True)
    G.compare_engines(hip, sca, f"{cfg} hip-vs-scalar", exact=name != "stableadamw")
    # bf16 add_(x, alpha=...): ATen's CPU kernel fuses `self + alpha * x` in fp32 in its vector body but
    # works in bf16 arithmetic (the product rounded on its own) in the scalar loop for the last
    # numel % 32 elements, so the reference differs from itself there.  The kernels follow the vector body.
    tail = 32 if (cfg in ADD_ALPHA and dtype != torch.float32) else 0
    G.compare_engines(hip, ref, f"{cfg} hip-vs-forloop", exact=False, body_only=tail)


@pytest.mark.parametrize("cfg", ["adamw", "lion", "stableadamw", "adan", "sgd_momentum", "radam", "ranger"])
def test_unaligned_buffers(cfg, hip_device):
    """Views that start 2 bytes (bf16) past a 16-byte boundary take the element-aligned vector path."""
    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    sizes = [5, 600, 9000]
    params, grads = draw(sizes, torch.bfloat16, 4, seed=5)
    guard = Guarded(hip_device)
    hip = hip_engine(name, params, hip_device, guard, offset=1, **hyper)
    assert all(p.data_ptr() % 16 != 0 for p in hip.params)
    sca = ScalarRun(name, [p.clone() for p in params], **hyper)
    for gs in grads:
        hip.step([guard(g, 3) for g in gs])
        sca.step([g.clone() for g in gs])
    torch.cuda.synchronize()
    guard.check()
    G.compare_engines(hip, sca, f"{cfg} unaligned", exact=name != "stableadamw")


@pytest.mark.parametrize("cfg", ["adamw", "lion", "stableadamw", "adan", "sgd_momentum", "radam", "ranger"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16], ids=["bf16", "fp32", "fp16"])
def test_gradient_release_with_accumulation(cfg, dtype, hip_device):
    """Per-tensor entry points in reverse order; 3 accumulate-only micro-steps, then a full one."""
    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    sizes = [3, 520, 8200, 20000]
    params, grads = draw(sizes, dtype, 8, seed=11)
    guard = Guarded(hip_device)
    hip = hip_engine(name, params, hip_device, guard, gradient_release=True, **hyper)
    sca = ScalarRun(name, [p.clone() for p in params], gradient_release=True, **hyper)
    for t, gs in enumerate(grads):
        hip.optimizer_accumulation = sca.optimizer_accumulation = (t + 1) % 4 != 0
        before = [p.clone() for p in hip.params]
        for i in reversed(range(len(sizes))):
            hip.step_param(i, guard(gs[i]))
            sca.step_param(i, gs[i].clone())
        if hip.optimizer_accumulation:
            for b, p in zip(before, hip.params):
                G.assert_bits_equal(p, b, f"{cfg} accumulate-only step {t} changed a parameter")
    torch.cuda.synchronize()
    guard.check()
    G.compare_engines(hip, sca, f"{cfg} release", exact=name != "stableadamw")


def test_baseline_config_adamw_fp32_mlp(hip_device):
    """The small fp32 benchmark configuration: AdamW fp32, 2 x [W1 1024x4096, b1 4096, W2 4096x1024, b2 1024], 10 steps, seed 0."""
    from hip_engine import HipRun

    shapes = [(1024, 4096), (4096,), (4096, 1024), (1024,)] * 2
    hyper = dict(lr=1e-3, betas=(0.9, 0.99), eps=1e-6, weight_decay=1e-2)
    gen = torch.Generator().manual_seed(0)
    params = [torch.randn(s, generator=gen) * 0.02 for s in shapes]
    hip = HipRun("adamw", [p.to(hip_device) for p in params], **hyper)
    sca = ScalarRun("adamw", [p.clone() for p in params], **hyper)
    ref = ForLoopRun("adamw", [p.clone() for p in params], **hyper)
    for _ in range(10):
        gs = [torch.randn(s, generator=gen) * 1e-3 for s in shapes]
        hip.step([g.to(hip_device) for g in gs])
        sca.step([g.clone() for g in gs])
        ref.step(gs)
    G.compare_engines(hip, sca, "C1 hip-vs-scalar", exact=True)
    G.compare_engines(hip, ref, "C1 hip-vs-forloop", exact=False)


def test_empty_and_changing_lists(hip_device):
    from hip_engine import HipRun
    from optimi_amd import cabi

    L = cabi.lib()
    grp = cabi.Group()
    none = cabi.ptr_array([])
    rc = L.optimi_hip_adam_multi(grp.handle, 0, none, none, none, none, none, cabi.i64_array([]), cabi.BF16,
                                 1e-3, 0.1, 0.9, 0.1, 0.99, 1e-6, cabi.UPDATE | cabi.KAHAN, None)
    assert rc == 0
    hyper = CONFIGS["adamw"]
    sizes = [0, 300, 0, 9000]
    params, grads = draw(sizes, torch.bfloat16, 6, seed=3)
    hip = HipRun("adamw", [p.to(hip_device) for p in params], **hyper)
    sca = ScalarRun("adamw", [p.clone() for p in params], **hyper)
    for t, gs in enumerate(grads):
        # a different subset has gradients each step, and gradients live at new addresses
        skip = {1} if t % 3 == 1 else ({3} if t % 3 == 2 else set())
        hip.step([None if i in skip else g.to(hip_device) for i, g in enumerate(gs)])
        sca.step([None if i in skip else g.clone() for i, g in enumerate(gs)])
    for i in (1, 3):
        G.assert_bits_equal(hip.params[i], sca.params[i], f"tensor {i}")
        G.assert_bits_equal(hip.state[i]["kahan_comp"], sca.state[i]["kahan_comp"], f"kahan {i}")


@pytest.mark.parametrize("cfg", ["adamw", "stableadamw", "adan"])
@pytest.mark.parametrize("n_tensors", [1, 2, 15, 16, 17, 40])
def test_list_lengths_around_the_kernel_argument_table(cfg, n_tensors, hip_device):
    """Lists of up to 16 tensors travel as a kernel argument and are searched by the workgroups;
    longer ones go through the chunk map in device memory.  Both must give the emulator's bits
    on either side of the switch, with empty tensors in the middle and at the end of the list
    (they own no chunk) and tensors of one tile, one chunk and several chunks."""
    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    pattern = [8193, 0, 700, 512, 0, 8192, 1, 20000, 3, 0]
    sizes = [pattern[i % len(pattern)] for i in range(n_tensors)]
    if n_tensors > 2:
        sizes[-1] = 0
    params, grads = draw(sizes, torch.bfloat16, 5, seed=21 + n_tensors)
    guard = Guarded(hip_device)
    hip = hip_engine(name, params, hip_device, guard, **hyper)
    sca = ScalarRun(name, [p.clone() for p in params], **hyper)
    for t, gs in enumerate(grads):
        skip = {0} if (t == 2 and n_tensors > 1) else set()  # the list changes length and shifts by one
        hip.step([None if i in skip else guard(g) for i, g in enumerate(gs)])
        sca.step([None if i in skip else g.clone() for i, g in enumerate(gs)])
    torch.cuda.synchronize()
    guard.check()
    G.compare_engines(hip, sca, f"{cfg} list of {n_tensors}", exact=name != "stableadamw")


@pytest.mark.parametrize("cfg", ["adamw", "lion", "stableadamw", "adan", "sgd_momentum", "ranger"])
@pytest.mark.parametrize("n_tensors", [5, 19])
def test_resident_hint_changes_nothing(cfg, n_tensors, hip_device):
    """A small list is read with streaming loads, the same list marked OPTIMI_RESIDENT with cached
    loads: two copies of the tile body in the kernel, one set of bits."""
    from hip_engine import HipRun

    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    sizes = SIZES[-n_tensors:]
    params, grads = draw(sizes, torch.bfloat16, 4, seed=31)
    warm = HipRun(name, [p.to(hip_device) for p in params], resident=True, **hyper)
    cold = HipRun(name, [p.to(hip_device) for p in params], **hyper)
    for gs in grads:
        warm.step([g.to(hip_device) for g in gs])
        cold.step([g.to(hip_device) for g in gs])
    torch.cuda.synchronize()
    G.compare_engines(cold, warm, f"{cfg} streaming vs cached loads", exact=True)


def test_rejected_arguments_on_device(hip_device):
    from optimi_amd import cabi

    L = cabi.lib()
    grp = cabi.Group()
    t = torch.zeros(64, dtype=torch.bfloat16, device=hip_device)
    a = t.data_ptr()
    args = (64, cabi.BF16, 1e-3, 0.1, 0.9, 0.1, 0.99, 1e-6, cabi.UPDATE | cabi.KAHAN, None)
    assert L.optimi_hip_adam_single(a + 1, a, a, a, a, *args) == -4        # not aligned to the element size
    assert L.optimi_hip_adam_single(a, a, a, a, None, *args) == -1         # Kahan buffer needed but NULL
    assert L.optimi_hip_adam_single(a, a, a, a, None, 64, cabi.BF16, 1e-3, 0.1, 0.9, 0.1, 0.99, 1e-6, cabi.UPDATE, None) == 0
    ptrs = cabi.ptr_array([a, None])
    rc = L.optimi_hip_adam_multi(grp.handle, 2, ptrs, ptrs, ptrs, ptrs, ptrs, cabi.i64_array([64, 64]), *args[1:])
    assert rc == -1
    rc = L.optimi_hip_adam_multi(grp.handle, 1, ptrs, ptrs, ptrs, ptrs, ptrs, cabi.i64_array([-5]), *args[1:])
    assert rc == -2
    rc = L.optimi_hip_stableadamw_single(grp.handle, a, a, a, a, a, 64, cabi.BF16, 1e-3, 0.1, 0.9, 0.1, 1e-2, 1e-6, 0.0,
                                         cabi.UPDATE | cabi.DECOUPLE_LR, None)
    assert rc == -7                                                        # DECOUPLE_LR needs max_lr > 0
    assert L.optimi_hip_copy_probe(a, a, 24, None) == -2
    torch.cuda.synchronize()


def test_copy_probe(hip_device):
    from optimi_amd import cabi

    src = torch.randint(0, 255, (1 << 20,), dtype=torch.uint8, device=hip_device)
    dst = torch.zeros_like(src)
    rc = cabi.lib().optimi_hip_copy_probe(dst.data_ptr(), src.data_ptr(), src.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(src, dst)


def test_stableadamw_gives_the_same_bits_on_every_run(hip_device):
    """The per-tensor sum behind StableAdamW's clipped learning rate is taken in a fixed order (a
    shuffle tree per wavefront, one partial per workgroup, the partials summed in index order by
    one workgroup per tensor) - no atomics - so runs on the same inputs agree bit for bit however
    the workgroups were scheduled, whole-list and per-tensor alike.  Sizes up to 20 M elements
    (40,000 partials for the largest tensor)."""
    from hip_engine import HipRun

    hyper = CONFIGS["stableadamw"]
    sizes = [20_000_003, 5_000_000, 70001, 8193, 513, 1] * 3  # 18 tensors: device tables
    params, grads = draw(sizes, torch.bfloat16, 3, seed=77)
    dev_grads = [[(g * 30).to(hip_device) for g in gs] for gs in grads]  # large gradients: the clipping is active

    def run(multi):
        r = HipRun("stableadamw", [p.to(hip_device) for p in params], multi=multi, **hyper)
        for gs in dev_grads:
            r.step(gs)
        torch.cuda.synchronize()
        return r

    first = run(True)
    for again in (run(True), run(True), run(False)):
        G.compare_engines(first, again, "StableAdamW run to run", exact=True)
