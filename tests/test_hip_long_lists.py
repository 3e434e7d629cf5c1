"""Lists and tensors too long for one grid.

A HIP grid holds fewer than 2^32 threads - 2^26 of the library's 64-lane workgroups, 64 GiB per
array.  A launch beyond that does not fail: the hardware runs the workgroup count modulo 2^26, so a
longer list would be stepped in part and nothing would say so.  The library therefore steps such a
list with several launches of whole chunks.  Two kinds of test:

* the split itself on small lists, with the number of workgroups per launch turned down to three
  chunks (``optimi_hip_launch_limit``): every optimizer, both kinds of table, mixed dtypes,
  per-tensor calls, StableAdamW's partial sums and the traffic probe - bit for bit what one launch
  gives;
* one tensor and one list that really are beyond 2^26 workgroups (68.7 GB per array, SGD without
  momentum so that two arrays suffice), against the closed form 1 - 0.5 * 1 = 0.5 in every element.
"""

import pytest
import torch

import golden_util as G
from hip_engine import HipRun
from optimi_amd import cabi
from test_hip_parity import CONFIGS, OPT_OF, SIZES, draw

pytestmark = pytest.mark.gpu

THREE_CHUNKS = 3 * 16  # workgroups


@pytest.fixture
def launch_limit():
    L = cabi.lib()
    before = L.optimi_hip_launch_limit(0)

    def set_limit(workgroups):
        L.optimi_hip_launch_limit(workgroups)

    yield set_limit
    L.optimi_hip_launch_limit(before)
    assert L.optimi_hip_launch_limit(0) == before


@pytest.mark.parametrize("cfg", ["adamw", "adam_l2", "lion", "stableadamw", "adan", "sgd_momentum", "radam", "ranger"])
@pytest.mark.parametrize("n_tensors", [5, 19])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_a_list_stepped_by_several_launches(cfg, n_tensors, dtype, hip_device, launch_limit):
    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    sizes = SIZES[-n_tensors:]  # up to 100,003 elements: 13 chunks in bf16, 25 in fp32
    params, grads = draw(sizes, dtype, 4, seed=41)
    L = cabi.lib()
    one = HipRun(name, [p.to(hip_device) for p in params], **hyper)
    n0 = L.optimi_hip_launch_count()
    for gs in grads:
        one.step([g.to(hip_device) for g in gs])
    n_one = L.optimi_hip_launch_count() - n0
    launch_limit(THREE_CHUNKS)
    many = HipRun(name, [p.to(hip_device) for p in params], **hyper)
    n0 = L.optimi_hip_launch_count()
    for gs in grads:
        many.step([g.to(hip_device) for g in gs])
    n_many = L.optimi_hip_launch_count() - n0
    torch.cuda.synchronize()
    assert n_many >= n_one + 4 * 5, (n_one, n_many)  # the split did happen
    G.compare_engines(one, many, f"{cfg} one launch vs several", exact=True)


@pytest.mark.parametrize("cfg", ["adamw", "stableadamw", "adan"])
def test_per_tensor_calls_and_mixed_lists_split_too(cfg, hip_device, launch_limit):
    hyper, name = CONFIGS[cfg], OPT_OF[cfg]
    sizes = [100003, 8193, 40000, 17, 65536]
    params, grads = draw(sizes, torch.bfloat16, 3, seed=43)
    params = [p.float() if i in (1, 3) else p for i, p in enumerate(params)]          # a mixed list
    grads = [[g.float() if i in (1, 3) else g for i, g in enumerate(gs)] for gs in grads]

    def run(multi):
        r = HipRun(name, [p.to(hip_device) for p in params], multi=multi, **hyper)
        for gs in grads:
            r.step([g.to(hip_device) for g in gs])
        torch.cuda.synchronize()
        return r

    whole_list, per_tensor = run(True), run(False)
    launch_limit(THREE_CHUNKS)
    whole_list_split, per_tensor_split = run(True), run(False)
    G.compare_engines(whole_list, whole_list_split, f"{cfg} mixed list", exact=True)
    G.compare_engines(per_tensor, per_tensor_split, f"{cfg} per tensor", exact=True)


def test_the_traffic_probe_splits_too(hip_device, launch_limit):
    L = cabi.lib()
    group = cabi.Group()
    gen = torch.Generator().manual_seed(5)
    n_tensors, words = 20, [4 * (1000 + 4099 * i) for i in range(20)]

    def arrays():
        return [[torch.randint(-2**31, 2**31 - 1, (w,), generator=gen, dtype=torch.int64).to(torch.int32).to(hip_device)
                 for w in words] for _ in range(3)]

    gen.manual_seed(5)
    a = arrays()
    gen.manual_seed(5)
    b = arrays()

    def probe(cols):
        table, keep = cabi.ptr_table([[t.data_ptr() for t in col] for col in cols])
        rc = L.optimi_hip_stream_probe(group.handle, n_tensors, table, cabi.i64_array([4 * w for w in words]), 3, 2, 0, cabi.PROBE_SCRAMBLE,
                                       torch.cuda.current_stream().cuda_stream)
        cabi.check(rc, "optimi_hip_stream_probe")

    probe(a)
    launch_limit(THREE_CHUNKS)
    probe(b)
    torch.cuda.synchronize()
    for col_a, col_b in zip(a, b):
        for x, y in zip(col_a, col_b):
            assert torch.equal(x, y)
    group.close()


# ---- really beyond one grid ----

BEYOND = ((1 << 26) // 16 + 5) * 8192 + 123  # bf16 elements: 2^22 + 5 chunks and a ragged tail, 68.7 GB per array


def _needs(bytes_needed):
    torch.cuda.empty_cache()  # what earlier tests left in torch's allocator counts as free
    free, _ = torch.cuda.mem_get_info()
    if free < bytes_needed:
        pytest.skip(f"needs {bytes_needed / 2**30:.0f} GiB of device memory, {free / 2**30:.0f} GiB are free")


def _all_equal(t, value, piece=1 << 30):
    for start in range(0, t.numel(), piece):
        if not bool((t[start:start + piece] == value).all()):
            return False
    return True


def test_one_tensor_beyond_the_grid_limit(hip_device):
    _needs(2 * 2 * BEYOND + (8 << 30))
    L = cabi.lib()
    p = torch.ones(BEYOND, dtype=torch.bfloat16, device=hip_device)
    g = torch.ones(BEYOND, dtype=torch.bfloat16, device=hip_device)
    n0 = L.optimi_hip_launch_count()
    #                            param         grad          momentum and Kahan buffers   lr   momentum, decay
    rc = L.optimi_hip_sgd_single(p.data_ptr(), g.data_ptr(), None, None, BEYOND, cabi.BF16, 0.5, 0.0, 0.0, cabi.UPDATE,
                                 torch.cuda.current_stream().cuda_stream)
    cabi.check(rc, "optimi_hip_sgd_single")
    torch.cuda.synchronize()
    assert L.optimi_hip_launch_count() - n0 == 2
    assert _all_equal(p, 0.5), "part of a tensor beyond 2^26 workgroups was not stepped"
    assert _all_equal(g, 1.0)


def test_a_list_beyond_the_grid_limit(hip_device):
    _needs(2 * 2 * BEYOND + (8 << 30))
    L = cabi.lib()
    group = cabi.Group()
    p = torch.ones(BEYOND, dtype=torch.bfloat16, device=hip_device)
    g = torch.ones(BEYOND, dtype=torch.bfloat16, device=hip_device)
    # 24 tensors laid over the two buffers: 23 of about 1.2 G elements each, of different sizes, and the rest
    cuts, pos = [], 0
    for i in range(23):
        n = 512 * (2_343_750 + 193 * i)  # multiples of 512 elements keep every piece on the 1 KiB tile grid
        cuts.append((pos, n))
        pos += n
    cuts.append((pos, BEYOND - pos))
    assert cuts[-1][1] > 1 << 31  # the last tensor alone has more than 2^31 elements
    ps = [p[a:a + n] for a, n in cuts]
    gs = [g[a:a + n] for a, n in cuts]
    n0 = L.optimi_hip_launch_count()
    rc = L.optimi_hip_sgd_multi(group.handle, len(ps), cabi.ptr_array(t.data_ptr() for t in ps),
                                cabi.ptr_array(t.data_ptr() for t in gs), None, None, cabi.i64_array([n for _, n in cuts]),
                                cabi.BF16, 0.5, 0.0, 0.0, cabi.UPDATE, torch.cuda.current_stream().cuda_stream)
    cabi.check(rc, "optimi_hip_sgd_multi")
    torch.cuda.synchronize()
    assert L.optimi_hip_launch_count() - n0 == 2
    assert _all_equal(p, 0.5), "part of a list beyond 2^26 workgroups was not stepped"
    group.close()
