"""The allocation-free StableAdamW entry point against the entry point it is a variant of.

``optimi_hip_stableadamw_single_noalloc`` keeps its reduction partials and per-tensor scalars in
a fixed device array of the library instead of a group's allocated workspace.  Both entry points
are called through the C ABI on identical inputs; every output buffer must match bit for bit.
The calls come in pairs, the second on a smaller tensor than the first, so that a result that
depended on what the previous call left in the shared array would show.
"""

import pytest
import torch

from optimi_amd import cabi

pytestmark = pytest.mark.gpu

DT = {torch.float32: cabi.F32, torch.bfloat16: cabi.BF16, torch.float16: cabi.F16}
NAMES = ("param", "grad", "exp_avg", "exp_avg_sq", "kahan_comp")


def _inputs(numel, dtype, device, seed, big_grad):
    gen = torch.Generator().manual_seed(seed)
    p = (torch.randn(numel, generator=gen) * 0.02).to(dtype)
    # gradients well above sqrt(exp_avg_sq) make the RMS exceed 1, so the clipped lr differs from lr
    g = (torch.randn(numel, generator=gen) * (3e-2 if big_grad else 1e-3)).to(dtype)
    m = (torch.randn(numel, generator=gen) * 1e-3).to(dtype)
    v = (torch.rand(numel, generator=gen) * 1e-6).to(dtype)
    k = (torch.randn(numel, generator=gen) * 1e-5).to(dtype)
    return [t.to(device) for t in (p, g, m, v, k)]


def _step(entry, group, bufs, numel, dtype, scalars, flags):
    L = cabi.lib()
    fn = getattr(L, entry)
    lead = (group.handle,) if group is not None else ()
    kahan = bufs[4].data_ptr() if (flags & cabi.KAHAN and dtype != torch.float32) else None
    rc = fn(*lead, bufs[0].data_ptr(), bufs[1].data_ptr(), bufs[2].data_ptr(), bufs[3].data_ptr(), kahan, numel, DT[dtype],
            *scalars, flags, torch.cuda.current_stream().cuda_stream)
    cabi.check(rc, entry)


def _compare(numel, dtype, device, seed, scalars, flags, group, big_grad=False):
    want = _inputs(numel, dtype, device, seed, big_grad)
    got = [t.clone() for t in want]
    _step("optimi_hip_stableadamw_single", group, want, numel, dtype, scalars, flags)
    _step("optimi_hip_stableadamw_single_noalloc", None, got, numel, dtype, scalars, flags)
    torch.cuda.synchronize()
    for name, a, b in zip(NAMES, got, want):
        view = torch.int32 if dtype == torch.float32 else torch.int16
        assert torch.equal(a.view(view), b.view(view)), f"{name} differs: numel={numel} dtype={dtype} flags={flags}"
    return want


#            lr    1-b1h  b2h    1-b2h  wd    eps   max_lr
SCALARS = (1e-3, 0.19, 0.98, 0.02, 1e-2, 1e-6, 0.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_two_calls_in_a_row_second_smaller(hip_device, dtype):
    group = cabi.Group()
    flags = cabi.KAHAN | cabi.UPDATE
    # 3 chunks and a ragged tail, then a tensor inside one tile: the second call reads fewer
    # partials than the first one wrote
    first = _compare(3 * 8192 + 1000 + 3, dtype, hip_device, 1, SCALARS, flags, group, big_grad=True)
    second = _compare(300, dtype, hip_device, 2, SCALARS, flags, group, big_grad=True)
    assert first[0].numel() > second[0].numel()
    # a third, larger call after the small one
    _compare(70_000, dtype, hip_device, 3, SCALARS, flags, group)
    group.close()


def test_variants_and_accumulate_only(hip_device):
    group = cabi.Group()
    dtype = torch.bfloat16
    decoupled = (1e-3, 0.19, 0.98, 0.02, 1e-5, 1e-6, 2e-3)
    for flags, scalars in ((cabi.UPDATE, SCALARS),                                  # no Kahan buffer
                           (cabi.KAHAN | cabi.UPDATE | cabi.DECOUPLE_LR, decoupled),  # fully decoupled decay
                           (cabi.KAHAN, SCALARS),                                   # accumulate-only: no reduction at all
                           (cabi.KAHAN | cabi.UPDATE, SCALARS[:4] + (0.0,) + SCALARS[5:])):  # no decay
        _compare(20_000, dtype, hip_device, 5, scalars, flags, group, big_grad=True)
        _compare(513, dtype, hip_device, 6, scalars, flags, group)
    group.close()


def test_large_tensor_then_small(hip_device):
    # a tensor the size of Llama-7B's down projection (4096 x 11008), then a norm weight
    group = cabi.Group()
    flags = cabi.KAHAN | cabi.UPDATE
    _compare(4096 * 11008, torch.bfloat16, hip_device, 7, SCALARS, flags, group, big_grad=True)
    _compare(4096, torch.bfloat16, hip_device, 8, SCALARS, flags, group, big_grad=True)
    group.close()


def test_limit_and_argument_errors(hip_device):
    L = cabi.lib()
    fn = L.optimi_hip_stableadamw_single_noalloc
    t = torch.zeros(16, dtype=torch.bfloat16, device=hip_device)
    a = t.data_ptr()
    stream = torch.cuda.current_stream().cuda_stream
    flags = cabi.KAHAN | cabi.UPDATE
    # one element past the limit of each dtype is rejected before anything is launched or read
    assert fn(a, a, a, a, a, 268435456 + 1, cabi.BF16, *SCALARS, flags, stream) == -8
    assert fn(a, a, a, a, a, 134217728 + 1, cabi.F32, *SCALARS, flags, stream) == -8
    assert b"OPTIMI_NOALLOC_MAX_NUMEL" in L.optimi_hip_error_string(-8)
    assert fn(None, a, a, a, a, 16, cabi.BF16, *SCALARS, flags, stream) == -1
    assert fn(a, a, a, a, a, -1, cabi.BF16, *SCALARS, flags, stream) == -2
    assert fn(a, a, a, a, a, 16, 9, *SCALARS, flags, stream) == -3
    assert fn(a, a, a, a, a, 16, cabi.BF16, 1e-3, 0.19, 0.98, 0.02, 1e-2, 1e-6, 0.0, flags | cabi.DECOUPLE_LR, stream) == -7
    assert fn(a, a, a, a, a, 0, cabi.BF16, *SCALARS, flags, stream) == 0
    torch.cuda.synchronize()
    assert float(t.float().abs().sum()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_step_really_clips(hip_device, dtype):
    """With gradients far above sqrt(exp_avg_sq) the RMS is well above 1, so the learning rate the step
    uses is lr / RMS: the parameter must move by clearly less than the same Adam step without clipping
    moves it (optimi_hip_adam_single on the same inputs and scalars, no decay in either).  A run in
    which the partial sums or the per-tensor scalars were not read back from the scratch would step
    with the plain lr - or with garbage - and fail here."""
    numel = 50_000
    scalars = SCALARS[:4] + (0.0,) + SCALARS[5:]  # no weight decay
    start = _inputs(numel, dtype, hip_device, 21, big_grad=True)
    clipped = [t.clone() for t in start]
    plain = [t.clone() for t in start]
    flags = cabi.UPDATE
    _step("optimi_hip_stableadamw_single_noalloc", None, clipped, numel, dtype, scalars, flags)
    L = cabi.lib()
    rc = L.optimi_hip_adam_single(plain[0].data_ptr(), plain[1].data_ptr(), plain[2].data_ptr(), plain[3].data_ptr(), None, numel,
                                  DT[dtype], *scalars[:6], flags | cabi.DECOUPLE_WD, torch.cuda.current_stream().cuda_stream)
    cabi.check(rc, "optimi_hip_adam_single")
    torch.cuda.synchronize()
    # the moments are the same step for both
    assert torch.equal(clipped[2], plain[2]) and torch.equal(clipped[3], plain[3])
    moved_clipped = (clipped[0].double() - start[0].double()).abs().mean().item()
    moved_plain = (plain[0].double() - start[0].double()).abs().mean().item()
    g, v_new = start[1].double(), clipped[3].double()
    rms = (g * g / v_new.clamp_min(1e-12)).mean().sqrt().item()
    assert rms > 2.0, rms
    ratio = moved_clipped / moved_plain
    if dtype == torch.float32:
        assert 0.7 / rms < ratio < 1.3 / rms, (moved_clipped, moved_plain, rms)
    else:  # a bf16 parameter moves in whole ulps, so only the direction of the effect is held
        assert 0.0 < ratio < 0.6, (moved_clipped, moved_plain, rms)


def test_no_device_memory_is_allocated(hip_device):
    """What the entry point is for: after a first call (which looks the scratch's address up) calls of
    any size below the limit leave the amount of free device memory exactly as it was - nothing is
    allocated, nothing is freed - whereas the variant with a group grows the group's workspace."""
    flags = cabi.KAHAN | cabi.UPDATE
    sizes = [300, 3 * 8192 + 1000, 1 << 20, 5_000_000, 40_000_000, 17]
    sets = {n: _inputs(n, torch.bfloat16, hip_device, 30 + i, big_grad=True) for i, n in enumerate(sizes)}
    _step("optimi_hip_stableadamw_single_noalloc", None, sets[300], 300, torch.bfloat16, SCALARS, flags)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        for n in sizes:
            _step("optimi_hip_stableadamw_single_noalloc", None, sets[n], n, torch.bfloat16, SCALARS, flags)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    # the same calls through a group do allocate (its workspace grows to the largest tensor's partials)
    group = cabi.Group()
    for n in sizes:
        _step("optimi_hip_stableadamw_single", group, sets[n], n, torch.bfloat16, SCALARS, flags)
    torch.cuda.synchronize()
    free_group, _ = torch.cuda.mem_get_info()
    assert free_group < free_after
    group.close()


def test_exactly_the_largest_tensor(hip_device):
    """OPTIMI_NOALLOC_MAX_NUMEL(bf16) = 2^28 elements: every one of the scratch's 524,288 partials is
    written and read; the result equals the group variant's."""
    numel = 268435456
    group = cabi.Group()
    gen = torch.Generator(device=hip_device).manual_seed(9)
    want = [torch.empty(numel, dtype=torch.float32, device=hip_device).normal_(0, s, generator=gen).bfloat16()
            for s in (0.02, 3e-2, 1e-3, 1e-3, 1e-5)]
    want[3].abs_().mul_(1e-3)
    got = [t.clone() for t in want]
    flags = cabi.KAHAN | cabi.UPDATE
    _step("optimi_hip_stableadamw_single", group, want, numel, torch.bfloat16, SCALARS, flags)
    _step("optimi_hip_stableadamw_single_noalloc", None, got, numel, torch.bfloat16, SCALARS, flags)
    torch.cuda.synchronize()
    for name, a, b in zip(NAMES, got, want):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"{name} differs at the size limit"
    group.close()
