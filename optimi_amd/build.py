"""In-tree build of the two native pieces.

* ``liboptimi_hip.so`` – the gfx950 kernels and the C ABI (hipcc, no torch).
* ``_C.*.so``          – the PyTorch-ROCm binding over that ABI (g++, host code only).

Both land next to this file so they travel with the source tree.  Run
``python -m optimi_amd.build`` to build them by hand.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "liboptimi_hip.so")
EXT_SUFFIX = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
BINDING_PATH = os.path.join(HERE, "_C" + EXT_SUFFIX)
ROCM_HOME = os.environ.get("ROCM_HOME", "/opt/rocm")

# -ffp-contract=off: the kernels spell out every fused multiply-add they want.
# packed-fp32-ops is switched off: hipcc must not form v_pk_*_f32 from the float code.
# -disable-vector-combine: that LLVM pass turns `pair * scalar_field` (a scalar read from the
# launch-scalars struct and splatted) into a two-float load that overlaps the next field; the
# overlapping loads then keep the optimizer from taking the struct apart, and the backend parks
# what is left of it in LDS - 768 to 1792 bytes per workgroup in every fp32 Adam, Adan and
# StableAdamW kernel, which costs a granule or two of the LDS budget that sets the occupancy
# and puts LDS reads into the element loops (fp32 AdamW over a cache-resident list: 74.5 us
# with the pass, 67.5 us without; the 16-bit kernels are unchanged within noise).
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-disable-vector-combine",
]


def _run(cmd: list[str]):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"build step failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    return proc


def build_lib(verbose: bool = False) -> str:
    hipcc = shutil.which("hipcc") or os.path.join(ROCM_HOME, "bin", "hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, f"-I{INCLUDE}", "-o", LIB_PATH, os.path.join(CSRC, "optimi_hip.hip")]
    if verbose:
        print(" ".join(cmd))
    _run(cmd)
    return LIB_PATH


def _binding_commands():
    import torch
    from torch.utils import cpp_extension as ce

    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{INCLUDE}", f"-I{ROCM_HOME}/include",
                                                     f"-I{sysconfig.get_paths()['include']}"]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    gxx = shutil.which("g++") or "g++"
    obj = os.path.join(CSRC, "torch_binding.o")
    compile_cmd = [
        gxx, "-O2", "-std=c++17", "-fPIC", "-c", "-Wno-deprecated-declarations",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-D_GLIBCXX_USE_CXX11_ABI={abi}", *inc, os.path.join(CSRC, "torch_binding.cpp"), "-o", obj,
    ]
    link_cmd = [
        gxx, "-shared", obj, "-o", BINDING_PATH,
        f"-L{HERE}", "-loptimi_hip", f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
        "-ltorch_python", f"-L{ROCM_HOME}/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}",
        f"-Wl,-rpath,{ROCM_HOME}/lib",
    ]
    return compile_cmd, link_cmd, obj


def build_binding(verbose: bool = False) -> str:
    """Compiles and links the binding; the kernel library must exist already (it is linked against)."""
    compile_cmd, link_cmd, obj = _binding_commands()
    try:
        for cmd in (compile_cmd, link_cmd):
            if verbose:
                print(" ".join(cmd))
            _run(cmd)
    finally:
        if os.path.exists(obj):
            os.remove(obj)
    return BINDING_PATH


def build_all(verbose: bool = False):
    """Both pieces; the binding's translation unit compiles while hipcc works on the kernels,
    and is linked once the library it links against is there."""
    from concurrent.futures import ThreadPoolExecutor

    compile_cmd, link_cmd, obj = _binding_commands()
    try:
        with ThreadPoolExecutor(max_workers=2) as pool:
            lib = pool.submit(build_lib, verbose)
            if verbose:
                print(" ".join(compile_cmd))
            binding = pool.submit(_run, compile_cmd)
            lib.result()
            binding.result()
        if verbose:
            print(" ".join(link_cmd))
        _run(link_cmd)
    finally:
        if os.path.exists(obj):
            os.remove(obj)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", LIB_PATH, BINDING_PATH, file=sys.stderr)
