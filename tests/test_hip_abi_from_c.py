"""The C ABI used from plain C: ``tests/native/abi_host.c`` has no PyTorch and no Python in it -
the HIP runtime for device memory, ``include/optimi_hip.h`` for the steps - and holds whole-list
and per-tensor steps of AdamW, Lion, Adan and SGD, bf16 + Kahan and fp32, to the scalar C emulator
bit for bit.  Compiled here with gcc (host code only, a second), run as a child process."""

import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ROCM = os.environ.get("ROCM_HOME", "/opt/rocm")


def compile_host(out):
    from oracle import scalar

    if not os.path.exists(scalar.LIB_PATH):  # the emulator the program links as its checker
        scalar.build()
    gcc = shutil.which("gcc") or "gcc"
    cmd = [gcc, "-O1", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", f"-I{ROCM}/include", f"-I{ROOT}/include",
           f"{ROOT}/tests/native/abi_host.c", "-o", out, f"-L{ROOT}/optimi_amd", "-loptimi_hip", f"-L{ROOT}/oracle",
           "-loptimi_ref", f"-L{ROCM}/lib", "-lamdhip64", "-lm", f"-Wl,-rpath,{ROOT}/optimi_amd", f"-Wl,-rpath,{ROOT}/oracle",
           f"-Wl,-rpath,{ROCM}/lib"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    return out


def test_a_plain_c_host_builds_against_the_header(tmp_path):
    compile_host(str(tmp_path / "abi_host"))


@pytest.mark.gpu
def test_a_plain_c_host_steps_and_matches_the_emulator(tmp_path):
    exe = compile_host(str(tmp_path / "abi_host"))
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "abi_host ok" in proc.stdout, proc.stdout
    assert proc.stdout.count(": ok") == 8, proc.stdout


@pytest.mark.gpu
def test_the_host_side_walked_from_c(tmp_path):
    """``abi_host paths``: lists that grow and shrink on one group, every whole-list entry point with
    one dtype and with a dtype per tensor, moved pointers, misaligned gradients, per-tensor StableAdamW
    on growing tensors, the probes, split launches.  Every call must succeed.  (The same program
    with the library's host code built under AddressSanitizer and UndefinedBehaviorSanitizer is how
    the host side was checked for memory errors; that build takes minutes and is not part of this run.)"""
    exe = compile_host(str(tmp_path / "abi_host"))
    proc = subprocess.run([exe, "paths"], capture_output=True, text=True, timeout=150)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "abi_host paths ok" in proc.stdout, proc.stdout
