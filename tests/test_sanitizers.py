"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (CPU only, no GPU, no Python
in the sanitized processes).

* The list-launch tables - argument validation, tensor table, chunk map, the search of the
  kernel-argument table and the tile arithmetic the kernels share - are plain C++ in
  ``optimi_amd/csrc/tables.h``; ``tests/native/table_fuzz.cpp`` drives them with adversarial lists.
* The scalar C emulator (``oracle/scalar_ref.c``), the checker every GPU parity test relies on, runs
  over exactly-sized heap buffers in ``oracle/sanitize_check.c``; the sanitized build must print
  what the plain build prints.
"""

import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SANITIZE = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-g"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")


def run(cmd, **kw):
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600, **kw)
    assert proc.returncode == 0, f"{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}"
    return proc


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_table_builder_fuzz_under_sanitizers(tmp_path):
    exe = str(tmp_path / "table_fuzz")
    run(["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", *SANITIZE, f"-I{ROOT}/include", f"-I{ROOT}/optimi_amd/csrc",
         "-o", exe, f"{ROOT}/tests/native/table_fuzz.cpp"])
    out = run([exe, "400"], env=ENV)
    assert "table_fuzz ok" in out.stdout and not out.stderr.strip(), out.stderr


@pytest.mark.skipif(shutil.which("gcc") is None or shutil.which("make") is None, reason="needs gcc and make")
def test_scalar_emulator_under_sanitizers(tmp_path):
    work = tmp_path / "oracle"
    work.mkdir()
    for name in ("Makefile", "scalar_ref.c", "sanitize_check.c"):
        shutil.copy(os.path.join(ROOT, "oracle", name), work / name)
    run(["make", "-C", str(work), "sanitize_check_san", "sanitize_check_plain"])
    san = run([str(work / "sanitize_check_san")], env=ENV)
    plain = run([str(work / "sanitize_check_plain")])
    assert not san.stderr.strip(), san.stderr
    lines = san.stdout.split()
    assert lines[0::2] == ["adam", "lion", "stableadamw", "adan", "sgd", "ranger"]
    assert san.stdout == plain.stdout
