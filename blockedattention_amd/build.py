"""Build recipe: ``python -m blockedattention_amd.build [lib|ext|all]``.

* ``lib`` -- the HIP kernels and the C ABI, compiled for gfx950 by hipcc into
  ``blockedattention_amd/lib/libblockedattn_hip.so``.  No torch involved.
* ``ext`` -- the torch binding ``blockAttention`` (same module and op names as
  the reference's extension), compiled by the host C++ compiler against
  libtorch and linked to the library above.  It contains no device code.

Everything is built in-tree so the shared objects travel with the source tree.
"""
import os
import shlex
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIBDIR = os.path.join(PKG, "lib")
OBJDIR = os.path.join(PKG, "lib", "obj")
LIB_PATH = os.path.join(LIBDIR, "libblockedattn_hip.so")
EXT_PATH = os.path.join(PKG, "blockAttention" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))

HIP_SOURCES = ["scheduler.hip", "gemm_softmax.hip", "onecall_kernel.hip", "tile_kernel.hip", "rowblock_kernel.hip", "rowpipe_kernel.hip", "softmax.hip", "gemm_generic.hip", "gemm_any16.hip", "attention.hip", "capi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
]


def _run(cmd, quiet=False):
    if not quiet:
        print("+", " ".join(shlex.quote(c) for c in cmd), flush=True)
    subprocess.check_call(cmd)


def build_lib(quiet=False, extra_flags=()):
    os.makedirs(OBJDIR, exist_ok=True)
    objs = [os.path.join(OBJDIR, s.replace(".hip", ".o")) for s in HIP_SOURCES]

    def compile_one(pair):
        src, obj = pair
        _run([HIPCC, *HIP_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj], quiet)

    with ThreadPoolExecutor(max_workers=min(len(objs), os.cpu_count() or 1)) as pool:
        list(pool.map(compile_one, zip(HIP_SOURCES, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs], quiet)
    return LIB_PATH


def build_ext(quiet=False):
    import torch
    from torch.utils import cpp_extension

    if not os.path.exists(LIB_PATH):
        build_lib(quiet)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"], "-isystem", "/opt/rocm/include",
            "-I", os.path.join(ROOT, "include")]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [
        os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
        "-DTORCH_EXTENSION_NAME=blockAttention", "-DTORCH_API_INCLUDE_EXTENSION_H",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        *inc, os.path.join(CSRC, "torch_binding.cpp"), "-o", EXT_PATH,
        "-L", torch_lib, "-L", LIBDIR, "-L", "/opt/rocm/lib",
        "-lblockedattn_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        "-lamdhip64",
        "-Wl,-rpath,$ORIGIN/lib", f"-Wl,-rpath,{torch_lib}", "-Wl,-rpath,/opt/rocm/lib",
    ]
    _run(cmd, quiet)
    return EXT_PATH


def build_all(quiet=False):
    build_lib(quiet)
    build_ext(quiet)


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    {"lib": build_lib, "ext": build_ext, "all": build_all}[what]()
