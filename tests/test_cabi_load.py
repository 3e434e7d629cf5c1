"""The C-ABI library loads without a GPU and exports every function include/optimi_hip.h
declares.  No compute entry point is called here."""

import ctypes
import os
import re

from optimi_amd import cabi

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "optimi_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(optimi_hip_\w+)\s*\(", text)))


def test_header_and_prototypes_agree():
    assert declared_functions() == sorted(cabi.PROTOTYPES)


def test_every_declared_symbol_is_exported():
    L = cabi.lib()
    for name in declared_functions():
        assert getattr(L, name) is not None, name


def test_error_strings_and_constants():
    L = cabi.lib()
    assert L.optimi_hip_version() >= 1000
    assert L.optimi_hip_error_string(0) == b"success"
    for code in range(-9, 0):
        msg = L.optimi_hip_error_string(code)
        assert msg.startswith(b"optimi_hip:"), (code, msg)
    assert L.optimi_hip_chunk_elems(cabi.BF16) == 8192
    assert L.optimi_hip_chunk_elems(cabi.F32) == 4096
    assert L.optimi_hip_chunk_elems(7) < 0
    # the flag values the Python side uses are the header's
    text = open(HEADER).read()
    for name, val in (("KAHAN", cabi.KAHAN), ("UPDATE", cabi.UPDATE), ("DECOUPLE_WD", cabi.DECOUPLE_WD),
                      ("ADAM_WD", cabi.ADAM_WD), ("DECOUPLE_LR", cabi.DECOUPLE_LR), ("RESIDENT", cabi.RESIDENT),
                      ("PROBE_SCRAMBLE", cabi.PROBE_SCRAMBLE)):
        assert re.search(rf"OPTIMI_{name}\s*=\s*{val}\b", text), name


def test_null_group_is_rejected_before_any_device_work():
    L = cabi.lib()
    assert L.optimi_hip_group_create(None) == -1
    assert L.optimi_hip_group_destroy(None) == 0
    nothing = (ctypes.c_void_p * 1)()
    sizes = (ctypes.c_int64 * 1)(0)
    rc = L.optimi_hip_adam_multi(None, 0, nothing, nothing, nothing, nothing, nothing, sizes, cabi.F32,
                                 1e-3, 0.1, 0.9, 0.1, 0.0, 1e-6, cabi.UPDATE, None)
    assert rc == -1
    # argument checks of the per-tensor entry points run before any launch
    assert L.optimi_hip_adam_single(None, None, None, None, None, -1, cabi.F32, 1e-3, 0.1, 0.9, 0.1, 0.0, 1e-6, 2, None) == -2
    assert L.optimi_hip_adam_single(None, None, None, None, None, 8, 9, 1e-3, 0.1, 0.9, 0.1, 0.0, 1e-6, 2, None) == -3
    assert L.optimi_hip_adam_single(None, None, None, None, None, 8, cabi.F32, 1e-3, 0.1, 0.9, 0.1, 0.0, 1e-6, 2, None) == -1
    assert L.optimi_hip_adam_single(None, None, None, None, None, 0, cabi.F32, 1e-3, 0.1, 0.9, 0.1, 0.0, 1e-6, 2, None) == 0
    assert L.optimi_hip_copy_probe(None, None, 16, None) == -1


def test_stream_probe_rejects_bad_mixes_before_any_device_work():
    L = cabi.lib()
    table, keep = cabi.ptr_table([[None]] * 7)
    sizes = cabi.i64_array([0])
    assert L.optimi_hip_stream_probe(None, 1, table, sizes, 5, 4, 0, 0, None) == -1          # no group
    fake = ctypes.c_void_p(1)  # never dereferenced: the mix is checked first
    for n_read, n_write in ((0, 0), (3, 0), (3, 4), (8, 2), (-1, 1)):
        assert L.optimi_hip_stream_probe(fake, 1, table, sizes, n_read, n_write, 0, 0, None) == -7, (n_read, n_write)
    assert L.optimi_hip_stream_probe(fake, 1, table, sizes, 5, 4, 52, 0, None) == -7          # more LDS than a workgroup may ask for
    assert L.optimi_hip_stream_probe(fake, 1, table, sizes, 5, 4, -1, 0, None) == -7
    assert L.optimi_hip_stream_probe(fake, -1, table, sizes, 5, 4, 0, 0, None) == -2
    assert L.optimi_hip_stream_probe(fake, 1, None, sizes, 5, 4, 0, 0, None) == -1
    assert L.optimi_hip_stream_probe(fake, 1, table, cabi.i64_array([24]), 5, 4, 0, 0, None) == -2   # not whole vectors
    assert L.optimi_hip_stream_probe(fake, 1, table, cabi.i64_array([32]), 5, 4, 0, 0, None) == -1   # null array with bytes
    off, keep2 = cabi.ptr_table([[4096 + 8]] * 7)
    assert L.optimi_hip_stream_probe(fake, 1, off, cabi.i64_array([32]), 5, 4, 0, 0, None) == -4     # off the 16-byte grid
    del keep, keep2


def test_noalloc_limit_matches_its_scratch():
    """A tensor of exactly OPTIMI_NOALLOC_MAX_NUMEL elements needs exactly as many pass-1 partials as the
    fixed scratch holds behind its 256-byte head: a chunk of 16 KiB per array is shared by 16 one-wavefront
    workgroups of 1 KiB, each of which leaves one double."""
    text = open(HEADER).read()
    scratch = re.search(r"#define OPTIMI_NOALLOC_SCRATCH_BYTES \((\d+)u \* (\d+)u \* (\d+)u \+ (\d+)u\)", text)
    a, b, c, head = (int(x) for x in scratch.groups())
    limits = re.search(r"#define OPTIMI_NOALLOC_MAX_NUMEL\(dtype\) \(\(dtype\) == OPTIMI_F32 \? \(int64_t\)(\d+) : \(int64_t\)(\d+)\)", text)
    max_f32, max_low = (int(x) for x in limits.groups())
    partials = (a * b * c + head - 256) // 8
    L = cabi.lib()
    for dtype, limit in ((cabi.F32, max_f32), (cabi.BF16, max_low), (cabi.F16, max_low)):
        chunk = L.optimi_hip_chunk_elems(dtype)
        assert limit % chunk == 0 and limit // chunk * 16 == partials, (dtype, limit, chunk, partials)


def test_the_limit_is_the_grid_limit_and_rounds_to_chunks():
    L = cabi.lib()  # no device is touched: the limit is a host-side variable
    hardware = L.optimi_hip_launch_limit(0)
    assert hardware == (1 << 26) - 16  # the largest whole number of chunks below 2^32 / 64 workgroups
    try:
        assert L.optimi_hip_launch_limit(50) == hardware
        assert L.optimi_hip_launch_limit(1) == 48       # rounded down to whole chunks
        assert L.optimi_hip_launch_limit(1 << 40) == 16  # at least one chunk
        assert L.optimi_hip_launch_limit(-1) == hardware  # never above the hardware's
        assert L.optimi_hip_launch_limit(0) == hardware
    finally:
        L.optimi_hip_launch_limit(-1)
