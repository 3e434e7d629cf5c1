"""The traffic probe (optimi_hip_stream_probe): the optimizers' launch without their arithmetic.
It is a measurement aid, so what is checked is that it touches exactly what it says.  Plain, it
leaves every array as it was.  With OPTIMI_PROBE_SCRAMBLE every element of the first n_write
arrays gets a known function of everything that was read (so a probe that skipped a load or a
store, and measured another mix, would be seen), the read-only arrays and everything around the
buffers stay as they were; one kernel per call, short lists and long ones alike."""

import pytest
import torch

from optimi_amd import cabi

pytestmark = pytest.mark.gpu

GUARD = 64  # 32-bit words of sentinel on each side of every buffer
SENTINEL = 0x5A5A5A5A
SALT = 0x9E3779B9 - (1 << 32)


def make(n_tensors, n_arrays, sizes, device, seed):
    gen = torch.Generator().manual_seed(seed)
    bufs, views = [], []
    for a in range(n_arrays):
        col_b, col_v = [], []
        for t in range(n_tensors):
            words = sizes[t] // 4
            buf = torch.full((words + 2 * GUARD,), SENTINEL, dtype=torch.int32, device=device)
            view = buf[GUARD:GUARD + words]
            view.copy_(torch.randint(-2**31, 2**31 - 1, (words,), generator=gen, dtype=torch.int64).to(torch.int32))
            col_b.append(buf)
            col_v.append(view)
        bufs.append(col_b)
        views.append(col_v)
    return bufs, views


@pytest.mark.parametrize("n_read,n_write", [(1, 1), (3, 2), (4, 2), (4, 3), (5, 4), (7, 6), (7, 7)])
@pytest.mark.parametrize("n_tensors", [1, 5, 40])
def test_probe_touches_what_it_says(hip_device, n_read, n_write, n_tensors):
    L = cabi.lib()
    # whole tiles (1 KiB), partial tiles, one vector, nothing at all, more than a chunk (16 KiB)
    pool = [16, 0, 1024, 1040, 16384, 16400, 48 * 1024 + 528, 512, 2048, 100000 // 16 * 16]
    sizes = [pool[(3 * i + n_read) % len(pool)] for i in range(n_tensors)]
    bufs, views = make(n_tensors, n_read, sizes, hip_device, seed=n_read * 100 + n_tensors)
    table, keep = cabi.ptr_table([[v.data_ptr() if v.numel() else None for v in col] for col in views])
    group = cabi.Group()
    stream = torch.cuda.current_stream().cuda_stream
    for granules, flags in ((0, 0), (9, cabi.PROBE_SCRAMBLE), (0, cabi.PROBE_SCRAMBLE | cabi.RESIDENT), (14, 0)):
        before = [[v.clone() for v in col] for col in views]
        launches = L.optimi_hip_launch_count()
        cabi.check(L.optimi_hip_stream_probe(group.handle, n_tensors, table, cabi.i64_array(sizes), n_read, n_write, granules,
                                             flags, stream), "optimi_hip_stream_probe")
        torch.cuda.synchronize()
        assert L.optimi_hip_launch_count() - launches == (1 if sum(sizes) else 0)
        for t in range(n_tensors):
            mix = torch.full_like(before[0][t], SALT)
            for a in range(n_read):
                mix ^= before[a][t]
            for a in range(n_read):
                buf, words = bufs[a][t], sizes[t] // 4
                assert bool((buf[:GUARD] == SENTINEL).all()) and bool((buf[GUARD + words:] == SENTINEL).all()), "write outside a buffer"
                want = before[a][t] ^ (mix + a) if (a < n_write and flags & cabi.PROBE_SCRAMBLE) else before[a][t]
                assert torch.equal(views[a][t], want), (a, t, flags)
    del keep
    group.close()
