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
    # the step really clipped: with lr' < lr the parameter moved less than the unclipped Adam step would move it
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
