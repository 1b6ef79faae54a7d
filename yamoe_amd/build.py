"""Builds the native parts in-tree:

  yamoe_amd/libyamoe_hip.so      the C-ABI library (hipcc, gfx950 only, no torch dependency)
  yamoe_amd/_yamoe_amd_ops.so    the torch op registration (host C++ only, links the library above)

Run as `python -m yamoe_amd.build`.  Both are plain compiler invocations so that the build works
without a GPU.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_obj")
LIB_HIP = os.path.join(HERE, "libyamoe_hip.so")
LIB_OPS = os.path.join(HERE, "_yamoe_amd_ops.so")

HIP_SOURCES = ["route.hip", "permute.hip", "gemm.hip", "gemm_async.hip", "gemm_f32.hip", "stream.hip", "subops.hip", "router.hip", "probe.hip", "plain.hip", "cabi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
    # packed fp32 VALU forms are switched off on purpose (they have produced silent wrong results)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the asynchronous-copy asm statements name M0 as clobbered; clang warns that M0 is a reserved register
    "-Wno-inline-asm",
] + os.environ.get("YAMOE_HIPCC_EXTRA", "").split()


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return r.stdout


def build_hip(verbose=True):
    os.makedirs(OBJ, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        out = _run([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            # the host pass does not know the packed-fp32 feature name; that warning is harmless
            lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip()]
            if lines:
                print("\n".join(lines))
        return obj

    with ThreadPoolExecutor(max_workers=min(11, len(HIP_SOURCES))) as ex:
        objs = list(ex.map(compile_one, HIP_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_HIP] + objs)
    if verbose:
        print("built", LIB_HIP)
    return LIB_HIP


def build_ops(verbose=True):
    import torch
    from torch.utils import cpp_extension

    inc = cpp_extension.include_paths()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-DTORCH_EXTENSION_NAME=_yamoe_amd_ops"]
    for i in inc:
        cmd += ["-isystem", i]
    cmd += ["-isystem", "/opt/rocm/include", "-I", sysconfig.get_paths()["include"],
            "-I", os.path.join(HERE, "..", "include")]
    cmd += [os.path.join(CSRC, "torch_binding.cpp"), "-o", LIB_OPS,
            "-L", HERE, "-l:libyamoe_hip.so", "-Wl,-rpath,$ORIGIN",
            "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip",
            "-Wl,-rpath," + torch_lib]
    _run(cmd)
    if verbose:
        print("built", LIB_OPS)
    return LIB_OPS


def build_all(verbose=True):
    build_hip(verbose)
    build_ops(verbose)


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "hip":
        build_hip()
    elif len(sys.argv) > 1 and sys.argv[1] == "ops":
        build_ops()
    else:
        build_all()
