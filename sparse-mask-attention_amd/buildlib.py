"""In-tree build of the native artefacts, for gfx950 only.

* ``libsma_hip.so``              the HIP kernels and the C ABI of ``include/sma.h``; compiled by
                                 ``hipcc --offload-arch=gfx950`` straight from ``csrc/*.hip``.
* ``sparse_attn_cuda.<abi>.so``  the pybind11 module that Python imports; host-only C++ compiled
                                 by ``g++`` against the PyTorch headers and linked to the library
                                 above (``$ORIGIN`` rpath).

The reference builds its extension through ``torch.utils.cpp_extension.CUDAExtension``
(``setup.py:35-45``) or the JIT ``load`` (``run.py:118-135``); on ROCm both would first translate
the sources with hipify, which is exactly what this build avoids: the sources are HIP already and
go to the compilers as they are.

* ``libsma_probe.so``            benchmark infrastructure, not the product: a pure stream of MFMAs that
                                 ``bench.py`` times as a yardstick (``benchprobe/mfma_probe.hip``).

All artefacts are written next to this file so that they travel with the source tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

LIB_NAME = "libsma_hip.so"
MODULE_NAME = "sparse_attn_cuda"
HIP_SOURCES = ["attn_fwd.hip", "attn_bwd.hip", "pack_mask.hip", "capi.hip"]
PROBE_DIR = os.path.join(HERE, "benchprobe")
PROBE_LIB_NAME = "libsma_probe.so"
GPU_ARCH = "gfx950"


def lib_path() -> str:
    return os.path.join(HERE, LIB_NAME)


def module_path() -> str:
    return os.path.join(HERE, MODULE_NAME + sysconfig.get_config_var("EXT_SUFFIX"))


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only target feature below and says so once per
    # pass; the message is harmless and only hides real diagnostics.
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed with exit code {proc.returncode}: {' '.join(cmd)}")


def probe_lib_path() -> str:
    return os.path.join(HERE, PROBE_LIB_NAME)


def hipcc_path() -> str:
    return shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")


# The device-code flags every HIP source of this package is compiled with (the ISA scan in the tests
# compiles with the same list).
HIPCC_FLAGS = [f"--offload-arch={GPU_ARCH}", "-O3", "-std=c++17", "-fno-finite-math-only",
               # keep the compiler from forming packed-FP32 VALU instructions
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               # the asynchronous-copy statements name m0, which they write, as clobbered; clang remarks
               # on every reserved register in a clobber list
               "-Wno-inline-asm",
               f"-I{INCLUDE}", f"-I{CSRC}"]


def build_hip_library() -> str:
    out = lib_path()
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-fPIC", "-shared"]
    cmd += [os.path.join(CSRC, s) for s in HIP_SOURCES]
    cmd += ["-o", out, f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}", "-Wl,-soname," + LIB_NAME]
    _run(cmd)
    return out


def build_python_module() -> str:
    import torch
    from torch.utils import cpp_extension as ce

    cxx = os.environ.get("CXX", "g++")
    out = module_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(ROCM, "include"), INCLUDE]
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={MODULE_NAME}",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-Wno-deprecated-declarations"]
    cmd += [f"-I{p}" for p in inc]
    cmd += [os.path.join(CSRC, "binding.cpp"), "-o", out,
            f"-L{HERE}", "-lsma_hip", "-Wl,-rpath,$ORIGIN",
            f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_python",
            f"-Wl,-rpath,{torch_lib}"]
    _run(cmd)
    return out


def build_probe_library() -> str:
    out = probe_lib_path()
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-fPIC", "-shared", f"-I{PROBE_DIR}",
                                           os.path.join(PROBE_DIR, "mfma_probe.hip"), "-o", out,
                                           f"-Wl,-rpath,{os.path.join(ROCM, 'lib')}", "-Wl,-soname," + PROBE_LIB_NAME]
    _run(cmd)
    return out


def build_all() -> None:
    build_hip_library()
    build_python_module()
    build_probe_library()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
