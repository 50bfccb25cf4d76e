"""Builds the native pieces in-tree:

  libfastmax_hip.so   the gfx950 kernels behind the C ABI of include/fastmax_amd.h
  fastmax_cuda*.so    the PyTorch C++ extension exporting forwardpass / backwardpass

`python -m fastmax_amd.build` compiles both; nothing is compiled at import time.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops off: scalar fp32 code must not be fused into v_pk_*_f32 on this hardware pool.  The
# feature switch acts on the device pass (a float2 multiply-add compiles to v_pk_fma_f32 without it and to
# two v_fma_f32 with it: tests/test_build_flags_cpu.py); the "not a recognized feature" warning hipcc
# prints for it comes from the host pass, which has no such feature, and is harmless.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        sys.stdout.write(proc.stdout)
        raise RuntimeError(f"build step failed ({proc.returncode}): {cmd[0]}")
    return proc.stdout


def _check_no_spills(remarks: str) -> None:
    """Every kernel must fit its registers: a build in which one of the matrix kernels spilled to
    scratch memory produced wrong accumulator values on the GPU, so a spill fails the build."""
    import re

    bad = []
    for block in re.split(r"remark: [^\n]*Function Name: ", remarks)[1:]:
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", block)
        if m and int(m.group(1)) > 0:
            bad.append(f"{block.splitlines()[0].strip()}: {m.group(1)} bytes/lane")
    if bad:
        raise RuntimeError("kernels spill registers to scratch memory:\n  " + "\n  ".join(bad))


def build_kernels() -> str:
    out = os.path.join(HERE, "libfastmax_hip.so")
    remarks = _run([HIPCC, *HIP_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-shared", f"-I{INCLUDE}", f"-I{CSRC}",
                    os.path.join(CSRC, "fm_api.hip"), "-o", out])
    _check_no_spills(remarks)
    return out


def extension_path() -> str:
    return os.path.join(HERE, "fastmax_cuda" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_extension() -> str:
    """The pybind11 module `fastmax_cuda` (host C++ only; it calls the C ABI)."""
    import torch
    from torch.utils import cpp_extension as ce

    out = extension_path()
    tdir = os.path.dirname(torch.__file__)
    inc = [f"-I{p}" for p in ce.include_paths(device_type="cuda")] + [
        f"-I{sysconfig.get_paths()['include']}", f"-I{INCLUDE}", "-I/opt/rocm/include"]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=fastmax_cuda", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *inc, os.path.join(CSRC, "fastmax_torch.cpp"), "-o", out,
           f"-L{HERE}", "-lfastmax_hip", f"-L{os.path.join(tdir, 'lib')}", "-ltorch", "-ltorch_cpu",
           "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{os.path.join(tdir, 'lib')}"]
    _run(cmd)
    return out


def build_all() -> None:
    build_kernels()
    build_extension()


if __name__ == "__main__":
    build_all()
