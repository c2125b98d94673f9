"""In-tree build of the two native pieces (run on a CPU-only machine; hipcc
cross-compiles for gfx950):

``libtorchex_scatter.so``  HIP kernels + C ABI (four translation units under
                           ``csrc/``), built with hipcc, no torch in it.
``scatter_ext*.so``        the PyTorch C++ extension module, built with the host
                           compiler against the torch headers; links to the
                           library above through ``$ORIGIN``.

``python torchex_amd/_build.py`` builds both (run it as a script: importing the
package needs the very files this module creates).
"""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
KERNEL_LIB = os.path.join(PKG, "libtorchex_scatter.so")
EXT_SUFFIX = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
EXT_LIB = os.path.join(PKG, "scatter_ext" + EXT_SUFFIX)
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

# packed-fp32 code generation is switched off for every HIP translation unit
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
KERNEL_SOURCES = ["plan_kernels.hip", "frontend_kernels.hip", "scatter_kernels.hip", "table_kernels.hip"]
OBJ_DIR = os.path.join(PKG, "_obj")


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels():
    """Compile the HIP translation units side by side, then link them into one library."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = []
    for name in KERNEL_SOURCES:
        obj = os.path.join(OBJ_DIR, os.path.splitext(name)[0] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I" + INCLUDE, "-c", os.path.join(CSRC, name), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        jobs.append((cmd, obj, subprocess.Popen(cmd)))
    for cmd, _, proc in jobs:
        if proc.wait() != 0:
            raise subprocess.CalledProcessError(proc.returncode, cmd)
    _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", KERNEL_LIB, *[obj for _, obj, _ in jobs]])
    return KERNEL_LIB


def build_ext():
    import torch
    from torch.utils import cpp_extension

    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    incs = cpp_extension.include_paths("cuda") + [sysconfig.get_paths()["include"], INCLUDE]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
        "-Wno-unused-function",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=scatter_ext",
        "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        *["-I" + p for p in incs],
        os.path.join(CSRC, "scatter_ext.cpp"),
        "-o", EXT_LIB,
        "-L" + PKG, "-ltorchex_scatter",
        "-L" + torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib,
    ]
    _run(cmd)
    return EXT_LIB


def build_all():
    build_kernels()
    build_ext()


def ensure_built():
    """Build what is missing (a fresh checkout has no shared objects: they are not
    tracked).  Used by the test suite, ``bench.py`` and the smoke entry point; importing
    ``torchex_amd`` itself never builds and raises if a piece is missing."""
    if not os.path.exists(KERNEL_LIB):
        build_kernels()
    if not os.path.exists(EXT_LIB):
        build_ext()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
